/*
 * TEST INFRASTRUCTURE - not part of the product. Only tests/ and bench.py's
 * cpu_baseline leg may load this.
 *
 * The loops Theano's C backend runs on the host for benchmark configurations
 * 1, 3, 4 and 5, restated node by node so that they can be timed beside the
 * GPU path (configuration 2 is oracle_careduce in careduce.c).  The reference
 * never fuses an Elemwise into a CAReduce on the CPU, so every configuration is
 * a chain of
 *   - Elemwise nodes: one loop nest per fused Composite, OpenMP
 *     "parallel for" when the node has >= 200000 elements
 *     (config.openmp_elemwise_minsize; theano/tensor/elemwise.py:1100-1102 for
 *     the contiguous path, theano/tensor/elemwise_cgen.py:406-409 for the
 *     outermost loop of the general path), typed temporaries per Composite
 *     statement (theano/scalar/basic.py:3796-3846);
 *   - CAReduce nodes: one accumulator per output, kept dimensions outermost,
 *     reduced dimensions innermost, no OpenMP
 *     (theano/tensor/elemwise.py:1384-1556, elemwise_cgen.py:465-527).
 * Intermediate arrays between nodes are materialised, as the reference's VM
 * does.  Per-element expressions follow theano/scalar/basic.py (Mod
 * :2119-2135, RightShift via >>, TrueDiv :1891-1915) and
 * theano/tensor/nnet/sigm.py:60-85.  Results are checked against the unfused
 * NumPy evaluation of the same graphs in tests/test_oracle_graph.py.
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

#define OMP_MIN 200000

/* numpy's half <-> float conversions (round to nearest even), bit-level */
static inline float h2f(uint16_t h) {
  const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1f, man = h & 0x3ffu, bits;
  if (exp == 0) {
    if (man == 0) {
      bits = sign;
    } else {
      int e = -1;
      do {
        ++e;
        man <<= 1;
      } while (!(man & 0x400u));
      bits = sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3ffu) << 13);
    }
  } else if (exp == 31) {
    bits = sign | 0x7f800000u | (man << 13);
  } else {
    bits = sign | ((exp + 112) << 23) | (man << 13);
  }
  float f;
  memcpy(&f, &bits, 4);
  return f;
}

static inline uint16_t f2h(float f) {
  uint32_t x;
  memcpy(&x, &f, 4);
  const uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
  const uint32_t absx = x & 0x7fffffffu;
  if (absx >= 0x7f800000u) return (uint16_t)(sign | 0x7c00u | (absx > 0x7f800000u ? 0x200u | ((absx >> 13) & 0x3ffu) : 0));
  if (absx >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u);          /* rounds to infinity */
  if (absx < 0x33000001u) return sign;                                 /* rounds to zero */
  int32_t e = (int32_t)(absx >> 23) - 127;
  uint32_t man = (absx & 0x7fffffu) | 0x800000u;
  int shift;
  uint32_t base;
  if (e < -14) {           /* subnormal half */
    shift = 13 + (-14 - e);
    base = 0;
  } else {
    shift = 13;
    base = (uint32_t)(e + 15) << 10;
    man &= 0x7fffffu;
  }
  uint32_t q = man >> shift;
  const uint32_t rem = man & ((1u << shift) - 1), half = 1u << (shift - 1);
  if (rem > half || (rem == half && (q & 1))) ++q;
  return (uint16_t)(sign | (base + q));
}

/* ---- configuration 1: Elemwise{Composite{(scalar_sigmoid(((i0 * i1) + i2)) * i1)}} --------
 * a and b are all-broadcast operands read once (elemwise.py:1097-1099); x and the output are
 * C-contiguous, so this is the contiguous fast path with one flat loop. */
void cpu_c1(const float* x, const float* a, const float* b, float* out, int64_t n) {
  const float av = a[0], bv = b[0];
#pragma omp parallel for if (n >= OMP_MIN)
  for (int64_t i = 0; i < n; ++i) {
    const float t0 = av * x[i];
    const float t1 = t0 + bv;
    const float t2 = t1 < -88.0f ? 0.0f : t1 > 15.0f ? 1.0f : 1.0f / (1.0f + expf(-t1));
    out[i] = t2 * x[i];
  }
}

/* ---- configuration 3, forward, as the Elemwise / CAReduce chain ------------------------------
 * max{axis=1} -> Elemwise{exp(i0 - i1)} -> Sum{axis=1, acc=float64} -> Elemwise{true_div}.
 * e is the materialised intermediate (R x C), rowmax and rowsum are (R,). */
void cpu_c3_chain(const float* x, float* out, float* e, float* rowmax, float* rowsum, int64_t R, int64_t C) {
  for (int64_t r = 0; r < R; ++r) {
    float acc = -INFINITY;
    const float* xr = x + r * C;
    for (int64_t c = 0; c < C; ++c) {
      const float v = xr[c];
      acc = v > acc ? v : (acc >= v ? acc : NAN);
    }
    rowmax[r] = acc;
  }
#pragma omp parallel for if (R * C >= OMP_MIN)
  for (int64_t r = 0; r < R; ++r) {
    const float m = rowmax[r];
    for (int64_t c = 0; c < C; ++c) e[r * C + c] = expf(x[r * C + c] - m);
  }
  for (int64_t r = 0; r < R; ++r) {
    double acc = 0.0;
    const float* er = e + r * C;
    for (int64_t c = 0; c < C; ++c) acc = acc + (double)er[c];
    rowsum[r] = (float)acc;
  }
#pragma omp parallel for if (R * C >= OMP_MIN)
  for (int64_t r = 0; r < R; ++r) {
    const float s = rowsum[r];
    for (int64_t c = 0; c < C; ++c) out[r * C + c] = e[r * C + c] / s;
  }
}

/* ---- configuration 3, forward, as the row loop of the Softmax op ------------------------------
 * theano/tensor/nnet/nnet.py:510-560 (contiguous branch): row maximum, exp(x - max) stored,
 * double sum, scale by 1 / sum; rows in sequence, no OpenMP. */
void cpu_c3_rowloop(const float* x, float* sm, int64_t R, int64_t C) {
  for (int64_t r = 0; r < R; ++r) {
    const float* xr = x + r * C;
    float* sr = sm + r * C;
    float row_max = xr[0];
    for (int64_t c = 1; c < C; ++c) row_max = xr[c] > row_max ? xr[c] : row_max;
    for (int64_t c = 0; c < C; ++c) sr[c] = xr[c] - row_max;
    for (int64_t c = 0; c < C; ++c) sr[c] = expf(sr[c]);
    double sum = 0.0;
    for (int64_t c = 0; c < C; ++c) sum += sr[c];
    const double sum_inv = 1.0 / sum;
    for (int64_t c = 0; c < C; ++c) sr[c] *= sum_inv;
  }
}

/* ---- configuration 4 ---------------------------------------------------------------------------
 * a, b: int32 (N, Ch, H, W) C-contiguous, read through dimshuffle(0, 2, 3, 1) views; bias (Ch,).
 * r: int32 (N, H, W, Ch) C-contiguous.  Loop order follows the output's strides
 * (make_reordered_loop), OpenMP on the outermost loop. */
static inline int32_t mod_py(int32_t x, int32_t y) {   /* Mod.c_code, integer branch: sign of the divisor */
  int32_t m = x % y;
  if (m != 0 && ((m < 0) != (y < 0))) m += y;
  return m;
}

void cpu_c4_elemwise(const int32_t* a, const int32_t* b, const int32_t* bias, int32_t* r, int64_t N, int64_t Ch,
                     int64_t H, int64_t Wd) {
  const int64_t HW = H * Wd;
#pragma omp parallel for if (N * Ch * HW >= OMP_MIN)
  for (int64_t n = 0; n < N; ++n)
    for (int64_t p = 0; p < HW; ++p)
      for (int64_t c = 0; c < Ch; ++c) {
        const int64_t src = (n * Ch + c) * HW + p;
        const int32_t av = a[src], bv = b[src];
        const int32_t t0 = av & bv;
        const int32_t t1 = av >> 3;
        const int32_t t2 = t0 ^ t1;
        const int32_t t3 = mod_py(t2, 97);
        r[(n * HW + p) * Ch + c] = t3 + bias[c];
      }
}

/* Sum{axis=(0, 1, 2), dtype=int64} of r (N*H*W, Ch): kept dimension outermost */
void cpu_c4_sum(const int32_t* r, int64_t* s, int64_t rows, int64_t Ch) {
  for (int64_t c = 0; c < Ch; ++c) {
    int64_t acc = 0;
    for (int64_t i = 0; i < rows; ++i) acc = acc + (int64_t)r[i * Ch + c];
    s[c] = acc;
  }
}

/* Elemwise{gt}(a, 0) -> bool array, then Any / All over it (two CAReduce nodes) */
void cpu_c4_anyall(const int32_t* a, uint8_t* pos, uint8_t* any_out, uint8_t* all_out, int64_t n) {
#pragma omp parallel for if (n >= OMP_MIN)
  for (int64_t i = 0; i < n; ++i) pos[i] = a[i] > 0;
  uint8_t acc = 0;
  for (int64_t i = 0; i < n; ++i) acc = acc || pos[i];
  *any_out = acc;
  acc = 1;
  for (int64_t i = 0; i < n; ++i) acc = acc && pos[i];
  *all_out = acc;
}

/* ---- configuration 5, forward ------------------------------------------------------------------
 * x, y: float16 (N, Ch, H, W); gamma, beta: float16 (Ch,).  Nodes: Cast{float32} (xf materialised)
 * -> Sum{(0,2,3), acc=float32} -> /M -> Elemwise{sqr(xf - mean)} (materialised) -> Sum -> /M ->
 * Elemwise{Cast{float16}(gamma*(xf-mean)/sqrt(var+eps)+beta)}.  xf and d are (N*Ch*H*W) float32
 * scratch arrays; mean and var are (Ch,). */
static void sum_over_n_hw(const float* v, float* s, int64_t N, int64_t Ch, int64_t HW) {
  for (int64_t c = 0; c < Ch; ++c) {
    float acc = 0.0f;
    for (int64_t n = 0; n < N; ++n) {
      const float* q = v + (n * Ch + c) * HW;
      for (int64_t p = 0; p < HW; ++p) acc = acc + q[p];
    }
    s[c] = acc;
  }
}

void cpu_c5_fwd(const uint16_t* x, const uint16_t* gamma, const uint16_t* beta, uint16_t* y, float* xf, float* d,
                float* mean, float* var, int64_t N, int64_t Ch, int64_t HW) {
  const int64_t n_all = N * Ch * HW;
  const float M = (float)(N * HW);
#pragma omp parallel for if (n_all >= OMP_MIN)
  for (int64_t i = 0; i < n_all; ++i) xf[i] = h2f(x[i]);
  sum_over_n_hw(xf, mean, N, Ch, HW);
  for (int64_t c = 0; c < Ch; ++c) mean[c] = mean[c] / M;
#pragma omp parallel for if (n_all >= OMP_MIN)
  for (int64_t n = 0; n < N; ++n)
    for (int64_t c = 0; c < Ch; ++c) {
      const float m = mean[c];
      for (int64_t p = 0; p < HW; ++p) {
        const int64_t i = (n * Ch + c) * HW + p;
        const float t = xf[i] - m;
        d[i] = t * t;
      }
    }
  sum_over_n_hw(d, var, N, Ch, HW);
  for (int64_t c = 0; c < Ch; ++c) var[c] = var[c] / M;
#pragma omp parallel for if (n_all >= OMP_MIN)
  for (int64_t n = 0; n < N; ++n)
    for (int64_t c = 0; c < Ch; ++c) {
      const float m = mean[c], g = h2f(gamma[c]), bt = h2f(beta[c]);
      const float sd = sqrtf(var[c] + 1e-5f);
      for (int64_t p = 0; p < HW; ++p) {
        const int64_t i = (n * Ch + c) * HW + p;
        y[i] = f2h(g * (xf[i] - m) / sd + bt);
      }
    }
}

/* the two conversions over arrays, for the test that compares them with NumPy's */
void cpu_h2f_array(const uint16_t* h, float* f, int64_t n) {
  for (int64_t i = 0; i < n; ++i) f[i] = h2f(h[i]);
}

void cpu_f2h_array(const float* f, uint16_t* h, int64_t n) {
  for (int64_t i = 0; i < n; ++i) h[i] = f2h(f[i]);
}

/* threads an OpenMP region of this library runs with (OMP_NUM_THREADS or the core count) */
#include <omp.h>
int cpu_omp_threads(void) { return omp_get_max_threads(); }

/* ---- configuration 3, forward + gradient of sum(out * y) with respect to x -------------------------
 * The forward chain of cpu_c3_chain, then the gradient graph as reverse mode builds it and
 * elementwise fusion partitions it (islands end at every CAReduce):
 *   t  = y * e / (s * s)                      Elemwise (OpenMP), materialised
 *   gs = -sum(t, 1)                           Sum, float64 accumulator, serial
 *   u  = (y / s + gs) * e                     Elemwise, materialised
 *   gm = -sum(u, 1)                           Sum, serial
 *   dx = u + eq(m, x) * gm                    Elemwise (gradient through max: positions equal to it)
 * out, dx: (R, C); e, t, u: (R, C) scratch; rowmax, rowsum, gs, gm: (R,). */
void cpu_c3_fwd_grad(const float* x, const float* y, float* out, float* dx, float* e, float* t, float* u,
                     float* rowmax, float* rowsum, float* gs, float* gm, int64_t R, int64_t C) {
  cpu_c3_chain(x, out, e, rowmax, rowsum, R, C);
#pragma omp parallel for if (R * C >= OMP_MIN)
  for (int64_t r = 0; r < R; ++r) {
    const float s = rowsum[r];
    for (int64_t c = 0; c < C; ++c) t[r * C + c] = y[r * C + c] * e[r * C + c] / (s * s);
  }
  for (int64_t r = 0; r < R; ++r) {
    double acc = 0.0;
    for (int64_t c = 0; c < C; ++c) acc = acc + (double)t[r * C + c];
    gs[r] = -(float)acc;
  }
#pragma omp parallel for if (R * C >= OMP_MIN)
  for (int64_t r = 0; r < R; ++r) {
    const float s = rowsum[r], g = gs[r];
    for (int64_t c = 0; c < C; ++c) u[r * C + c] = (y[r * C + c] / s + g) * e[r * C + c];
  }
  for (int64_t r = 0; r < R; ++r) {
    double acc = 0.0;
    for (int64_t c = 0; c < C; ++c) acc = acc + (double)u[r * C + c];
    gm[r] = -(float)acc;
  }
#pragma omp parallel for if (R * C >= OMP_MIN)
  for (int64_t r = 0; r < R; ++r) {
    const float m = rowmax[r], g = gm[r];
    for (int64_t c = 0; c < C; ++c) dx[r * C + c] = u[r * C + c] + (x[r * C + c] == m ? 1.0f : 0.0f) * g;
  }
}

/* ---- configuration 5, gradients of sum(y * g) with respect to x, gamma, beta ----------------------
 * Forward statistics as in cpu_c5_fwd (xf, mean, d = sqr(xf - mean), var), then with
 * std = sqrt(var + eps), D = xf - mean, G = cast(g, float32):
 *   dbeta  = sum(G)                            Sum per channel, float64 accumulator (float32 input), serial
 *   sgd    = sum(G * D)                        Elemwise product materialised in d, then Sum
 *   dgamma = sgd / std
 *   dvar   = -gamma * sgd / (std * std) / (2 * std)                                  per channel
 *   dd     = G * gamma / std + 2 * D * dvar / M                                      Elemwise, materialised
 *   dmean  = -sum(dd)                          Sum
 *   dx     = cast(dd + dmean / M, float16)     Elemwise
 * xf, gf, d: (N*Ch*HW) float32 scratch; per-channel arrays of Ch floats. */
static void sum64_over_n_hw(const float* v, float* s, int64_t N, int64_t Ch, int64_t HW) {
  for (int64_t c = 0; c < Ch; ++c) {
    double acc = 0.0;
    for (int64_t n = 0; n < N; ++n) {
      const float* q = v + (n * Ch + c) * HW;
      for (int64_t p = 0; p < HW; ++p) acc = acc + (double)q[p];
    }
    s[c] = (float)acc;
  }
}

void cpu_c5_grad(const uint16_t* x, const uint16_t* gamma, const uint16_t* g, uint16_t* dx, uint16_t* dgamma,
                 uint16_t* dbeta, float* xf, float* gf, float* d, float* mean, float* var, float* tmp,
                 int64_t N, int64_t Ch, int64_t HW) {
  const int64_t n_all = N * Ch * HW;
  const float M = (float)(N * HW);
#pragma omp parallel for if (n_all >= OMP_MIN)
  for (int64_t i = 0; i < n_all; ++i) xf[i] = h2f(x[i]);
  sum_over_n_hw(xf, mean, N, Ch, HW);
  for (int64_t c = 0; c < Ch; ++c) mean[c] = mean[c] / M;
#pragma omp parallel for if (n_all >= OMP_MIN)
  for (int64_t n = 0; n < N; ++n)
    for (int64_t c = 0; c < Ch; ++c)
      for (int64_t p = 0; p < HW; ++p) {
        const int64_t i = (n * Ch + c) * HW + p;
        const float t = xf[i] - mean[c];
        d[i] = t * t;
      }
  sum_over_n_hw(d, var, N, Ch, HW);
  for (int64_t c = 0; c < Ch; ++c) var[c] = sqrtf(var[c] / M + 1e-5f);   /* var now holds std */
#pragma omp parallel for if (n_all >= OMP_MIN)
  for (int64_t i = 0; i < n_all; ++i) gf[i] = h2f(g[i]);
  sum64_over_n_hw(gf, tmp, N, Ch, HW);                                     /* tmp = dbeta */
  for (int64_t c = 0; c < Ch; ++c) dbeta[c] = f2h(tmp[c]);
#pragma omp parallel for if (n_all >= OMP_MIN)
  for (int64_t n = 0; n < N; ++n)
    for (int64_t c = 0; c < Ch; ++c)
      for (int64_t p = 0; p < HW; ++p) {
        const int64_t i = (n * Ch + c) * HW + p;
        d[i] = gf[i] * (xf[i] - mean[c]);
      }
  sum64_over_n_hw(d, tmp, N, Ch, HW);                                      /* tmp = sum(G * D) */
  for (int64_t c = 0; c < Ch; ++c) {
    const float sd = var[c], gm = h2f(gamma[c]);
    dgamma[c] = f2h(tmp[c] / sd);
    tmp[c] = -gm * tmp[c] / (sd * sd) / (2.0f * sd);                       /* tmp = dvar */
  }
#pragma omp parallel for if (n_all >= OMP_MIN)
  for (int64_t n = 0; n < N; ++n)
    for (int64_t c = 0; c < Ch; ++c) {
      const float sd = var[c], gm = h2f(gamma[c]), dv = tmp[c], m = mean[c];
      for (int64_t p = 0; p < HW; ++p) {
        const int64_t i = (n * Ch + c) * HW + p;
        d[i] = gf[i] * gm / sd + 2.0f * (xf[i] - m) * dv / M;
      }
    }
  sum64_over_n_hw(d, mean, N, Ch, HW);                                     /* mean now holds sum(dd) */
#pragma omp parallel for if (n_all >= OMP_MIN)
  for (int64_t n = 0; n < N; ++n)
    for (int64_t c = 0; c < Ch; ++c) {
      const float dm = -mean[c] / M;
      for (int64_t p = 0; p < HW; ++p) {
        const int64_t i = (n * Ch + c) * HW + p;
        dx[i] = f2h(d[i] + dm);
      }
    }
}

/* ---- configuration 2 with OpenMP over the outputs: NOT the reference's behaviour ------------------
 * The reference's CAReduce loops carry no OpenMP pragma (theano/tensor/elemwise_cgen.py:465-527).
 * These variants only show what the same host could do with all its cores: rows (axis 1) or
 * blocks of columns (axis 0) are spread over threads, each output still accumulated in order
 * in float64; the sum over all axes adds per-row partial sums, so its rounding may differ from
 * the serial loop's in the last place.  which: 0 sum axis 1, 1 max axis 1, 2 sum axis 0,
 * 3 sum of everything (out[0]), 4 prod axis 1. */
void cpu_c2_parallel(const float* x, float* out, int64_t R, int64_t C, int which) {
  if (which == 0 || which == 1 || which == 4) {
#pragma omp parallel for
    for (int64_t r = 0; r < R; ++r) {
      const float* q = x + r * C;
      if (which == 1) {
        float acc = -INFINITY;
        for (int64_t c = 0; c < C; ++c) acc = q[c] > acc ? q[c] : (acc >= q[c] ? acc : NAN);
        out[r] = acc;
      } else {
        double acc = which == 0 ? 0.0 : 1.0;
        if (which == 0)
          for (int64_t c = 0; c < C; ++c) acc = acc + (double)q[c];
        else
          for (int64_t c = 0; c < C; ++c) acc = acc * (double)q[c];
        out[r] = (float)acc;
      }
    }
  } else if (which == 2) {
    enum { CB = 256 };
#pragma omp parallel for
    for (int64_t c0 = 0; c0 < C; c0 += CB) {
      double acc[CB];
      const int64_t n = C - c0 < CB ? C - c0 : CB;
      for (int64_t c = 0; c < n; ++c) acc[c] = 0.0;
      for (int64_t r = 0; r < R; ++r)
        for (int64_t c = 0; c < n; ++c) acc[c] = acc[c] + (double)x[r * C + c0 + c];
      for (int64_t c = 0; c < n; ++c) out[c0 + c] = (float)acc[c];
    }
  } else {
    double total = 0.0;
#pragma omp parallel for reduction(+ : total)
    for (int64_t r = 0; r < R; ++r) {
      double acc = 0.0;
      for (int64_t c = 0; c < C; ++c) acc = acc + (double)x[r * C + c];
      total += acc;
    }
    out[0] = (float)total;
  }
}
