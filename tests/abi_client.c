/*
 * A host written in plain C against include/thx_hip.h: the same calls a cgo / JNI / ctypes
 * binding makes.  It builds out = a * x + b (a and b host scalars travelling by value, x a
 * matrix read through a transposed view) and checks the result.
 *
 *   abi_client dry    plans and compiles for gfx950 without a device
 *   abi_client        runs on device 0 and verifies every element
 */
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "thx_hip.h"

/* The functor contract of kernels/thx_elemwise.h, written by hand for z = a * x + b. */
static const char* FUNCTOR =
    "struct AxPlusB {\n"
    "  enum { NIN = 3, NOUT = 1, NOPS = 4 };\n"
    "  template <int V> struct Regs { thx::Vec<thx_f32, V> i0; thx::Vec<thx_f32, V> i1; thx::Vec<thx_f32, V> i2;\n"
    "                                 thx::Vec<thx_f32, V> o0; };\n"
    "  template <int V, class A> THX_DEV static void load(const A& a, Regs<V>& r) {\n"
    "    a.template ld<0>(r.i0); a.template ld<1>(r.i1); a.template ld<2>(r.i2);\n"
    "  }\n"
    "  template <int V> THX_DEV static void compute(Regs<V>& r) {\n"
    "#pragma unroll\n"
    "    for (int k = 0; k < V; ++k) r.o0.v[k] = r.i0.v[k] * r.i1.v[k] + r.i2.v[k];\n"
    "  }\n"
    "  template <int V, class A> THX_DEV static void store(const A& a, const Regs<V>& r) { a.template st<3>(r.o0); }\n"
    "};\n";

#define CHECK(call)                                                                 \
  do {                                                                              \
    int rc_ = (call);                                                               \
    if (rc_ != THX_OK) {                                                            \
      fprintf(stderr, "%s failed (%d): %s\n", #call, rc_, thx_last_error());        \
      return 1;                                                                     \
    }                                                                               \
  } while (0)

static thx_array matrix(void* base, int dtype, int64_t rows, int64_t cols, int64_t row_stride, int64_t col_stride) {
  thx_array a;
  memset(&a, 0, sizeof a);
  a.base = base;
  a.nd = 2;
  a.dtype = dtype;
  a.shape[0] = rows;
  a.shape[1] = cols;
  a.strides_bytes[0] = row_stride;
  a.strides_bytes[1] = col_stride;
  return a;
}

int main(int argc, char** argv) {
  const int dry = argc > 1 && strcmp(argv[1], "dry") == 0;
  enum { R = 300, C = 257 };
  const int32_t dtypes[4] = {THX_F32, THX_F32, THX_F32, THX_F32};
  float a = 1.5f, b = -0.25f;
  thx_elemwise* op = NULL;
  CHECK(thx_elemwise_new(FUNCTOR, "AxPlusB", 3, 1, dtypes, &op));

  float* host = (float*)malloc(sizeof(float) * R * C);
  float* back = (float*)malloc(sizeof(float) * R * C);
  for (int i = 0; i < R * C; ++i) host[i] = (float)(i % 1000) * 0.001f;
  void *dx = NULL, *dz = NULL;
  if (!dry) {
    CHECK(thx_init(0));
    CHECK(thx_alloc(sizeof(float) * R * C, &dx));
    CHECK(thx_alloc(sizeof(float) * R * C, &dz));
    CHECK(thx_h2d(dx, host, sizeof(float) * R * C));
  }
  /* x is stored (C, R); the operation reads its transpose: a view, no copy */
  thx_array ins[3], out;
  ins[0] = matrix(&a, THX_F32 | THX_HOST_SCALAR, 1, 1, 4, 4);
  ins[1] = matrix(dx, THX_F32, R, C, 4, 4 * R);
  ins[2] = matrix(&b, THX_F32 | THX_HOST_SCALAR, 1, 1, 4, 4);
  out = matrix(dz, THX_F32, R, C, 4 * C, 4);
  CHECK(thx_elemwise_call(op, ins, &out, THX_BROADCAST | (dry ? THX_DRY_RUN : 0)));
  printf("plan: %s\n", thx_last_plan());
  if (!dry) {
    CHECK(thx_d2h(back, dz, sizeof(float) * R * C));
    for (int r = 0; r < R; ++r)
      for (int c = 0; c < C; ++c) {
        /* the device contracts a * x + b into one fused multiply-add: equal up to the last place */
        const float want = a * host[c * R + r] + b;
        if (fabsf(back[r * C + c] - want) > 1e-6f * (1.0f + fabsf(want))) {
          fprintf(stderr, "mismatch at (%d, %d): %g != %g\n", r, c, back[r * C + c], want);
          return 1;
        }
      }
    /* a shape error is reported, not launched */
    ins[1].shape[0] = R - 1;
    if (thx_elemwise_call(op, ins, &out, THX_BROADCAST) != THX_ERR_SHAPE) {
      fprintf(stderr, "expected THX_ERR_SHAPE\n");
      return 1;
    }
    CHECK(thx_free(dx));
    CHECK(thx_free(dz));
  }
  CHECK(thx_elemwise_free(op));
  free(host);
  free(back);
  printf("ok\n");
  return 0;
}
