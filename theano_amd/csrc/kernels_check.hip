// Build-time compile check of the run-time kernel templates: the headers under
// kernels/ are instantiated with two sample functors (the shapes the Python code
// generator emits) for every kernel family and compiled for gfx950. Nothing in
// this file is linked into the library.
#include <hip/hip_runtime.h>

#include "kernels/thx_common.h"
#include "kernels/thx_special.h"
#include "kernels/thx_reduce.h"
#include "kernels/thx_elemwise.h"
#include "kernels/thx_rowchain.h"

struct CheckF {
  enum { NIN = 2, NOUT = 1, NOPS = 3 };
  template <int V> struct Regs { thx::Vec<thx_f16, V> i0; thx::Vec<thx_f32, V> i1; thx::Vec<thx_f32, V> o0; };
  template <int V, class A> THX_DEV static void load(const A& a, Regs<V>& r) { a.template ld<0>(r.i0); a.template ld<1>(r.i1); }
  THX_DEV static void apply(const thx_f32 i0, const thx_f32 i1, thx_f32& o0) { o0 = i0 * i1 + expf(i0); }
  template <int V> THX_DEV static void compute(Regs<V>& r) {
#pragma unroll
    for (int k = 0; k < V; ++k) { thx_f32 t; apply((thx_f32)r.i0.v[k], (thx_f32)r.i1.v[k], t); r.o0.v[k] = (thx_f32)t; }
  }
  template <int V, class A> THX_DEV static void store(const A& a, const Regs<V>& r) { a.template st<2>(r.o0); }
};

struct CheckR {
  enum { NIN = 1, NOUT = 2, NEX = 1 };
  struct Acc { thx_f64 a0; thx_f32 a1; };
  template <int V> struct Regs { thx::Vec<thx_f32, V> i0; };
  THX_DEV static void init(Acc& a) { a.a0 = 0.0; a.a1 = -INFINITY; }
  template <int V, class A> THX_DEV static void load(const A& a, Regs<V>& r) { a.template ld<0>(r.i0); }
  THX_DEV static void pre(const thx_f32 i0, Acc& v) { v.a0 = (thx_f64)i0; v.a1 = i0; }
  THX_DEV static void comb(Acc& a, const Acc& b) {
    a.a0 = a.a0 + b.a0;
    a.a1 = ((b.a1) > (a.a1) ? (b.a1) : ((a.a1) >= (b.a1) ? (a.a1) : NAN));
  }
  template <int V> THX_DEV static void accum(Acc& s, const Regs<V>& r) {
#pragma unroll
    for (int k = 0; k < V; ++k) { Acc t; pre((thx_f32)r.i0.v[k], t); comb(s, t); }
  }
  template <int V> THX_DEV static void accum_lanes(Acc* s, const Regs<V>& r) {
#pragma unroll
    for (int k = 0; k < V; ++k) { Acc t; pre((thx_f32)r.i0.v[k], t); comb(s[k], t); }
  }
  THX_DEV static Acc shfl_xor(const Acc& a, int m) { Acc r; r.a0 = thx::shfl_xor_t(a.a0, m); r.a1 = thx::shfl_xor_t(a.a1, m); return r; }
  template <class O> THX_DEV static void post(const O& o, long long idx, const Acc& a) {
    ((thx_f32*)o.ptr[0])[idx] = (thx_f32)a.a0;
    ((thx_f32*)o.ptr[1])[idx] = (thx_f32)a.a1 / *(const thx_f32*)&o.ex[0];
  }
};

// an elementwise functor with an attached reduction of its result (permuted-read kernel, reducing variant)
struct CheckFR : CheckF {
  typedef CheckR Red;
  template <int V, class AccT> THX_DEV static void red_lanes(AccT* acc, const Regs<V>& r) {
#pragma unroll
    for (int k = 0; k < V; ++k) { Red::Acc t; Red::pre((thx_f32)r.o0.v[k], t); Red::comb(acc[k], t); }
  }
};

struct PlanEw1 { typedef int IT; enum { ND = 1, VEC = 4, UNR = 2, BLOCK = 256, GS = 1, UA = 1, RAG = 0 }; static constexpr unsigned long long NT = 1ull;
  static constexpr int mode(int i) { constexpr int m[] = {0, 3, 0}; return m[i]; }
  static constexpr int sclass(int i, int d) { constexpr int m[][1] = {{1}, {0}, {1}}; return m[i][d]; }
  static constexpr int alias(int i) { constexpr int m[] = {0, 1, 0}; return m[i]; } };
struct PlanEw3 { typedef long long IT; enum { ND = 3, VEC = 2, UNR = 1, BLOCK = 256, GS = 0, UA = 1, RAG = 1 }; static constexpr unsigned long long NT = 1ull;
  static constexpr int mode(int i) { constexpr int m[] = {2, 1, 0}; return m[i]; }
  static constexpr int sclass(int i, int d) { constexpr int m[][3] = {{2, 2, 2}, {0, 1, 0}, {2, 2, 1}}; return m[i][d]; }
  static constexpr int alias(int i) { constexpr int m[] = {0, 1, 2}; return m[i]; } };
struct PlanRow { typedef int IT; enum { NK = 2, VEC = 4, UNR = 4, NACC = 2, BLOCK = 256, TPR = 256, RA2 = 1, TICKET = 0, GS = 1, XCD = 0, UA = 0 }; static constexpr unsigned long long NT = 0ull;
  static constexpr int mode(int i) { constexpr int m[] = {0}; return m[i]; }
  static constexpr int sclass(int i, int w) { constexpr int m[][2] = {{2, 1}}; return m[i][w]; } };
struct PlanRowS { typedef int IT; enum { NK = 1, VEC = 1, UNR = 1, NACC = 1, BLOCK = 256, TPR = 16, RA2 = 0, TICKET = 0, GS = 0, XCD = 1, UA = 1 }; static constexpr unsigned long long NT = 1ull;
  static constexpr int mode(int i) { constexpr int m[] = {2}; return m[i]; }
  static constexpr int sclass(int i, int w) { constexpr int m[][2] = {{0, 2}}; return m[i][w]; } };
struct PlanCol { typedef int IT; enum { NK = 1, VEC = 4, UNR = 4, BLOCK = 256, TX = 64, RR2 = 1, TICKET = 0, GS = 1, UA = 1 }; static constexpr unsigned long long NT = 1ull;
  static constexpr int mode(int i) { constexpr int m[] = {0}; return m[i]; } };
struct PlanStrip { typedef int IT; enum { VEC = 4, COLS = 3, BLOCK = 256, UA = 1 }; static constexpr unsigned long long NT = 1ull;
  static constexpr int mode(int i) { constexpr int m[] = {0}; return m[i]; } };
struct PlanGen { typedef int IT; enum { NK = 3, NR = 3, BLOCK = 256, TPR = 64, GS = 1, UA = 0 }; static constexpr unsigned long long NT = 0ull;
  static constexpr int mode(int i) { constexpr int m[] = {2}; return m[i]; } };

struct PlanTr { typedef int IT; enum { ND = 3, TT = 64, TI = 32, TV = 4, BLOCK = 256, NTR = 1, ESZ = 2, RED = 0, NBUF = 2, PERSIST = 1 }; static constexpr unsigned long long NT = 0ull;
  static constexpr int mode(int i) { constexpr int m[] = {2, 0, 0}; return m[i]; }
  static constexpr int slot(int i) { constexpr int m[] = {0, -1, -1}; return m[i]; } };
struct PlanTrRed { typedef int IT; enum { ND = 3, TT = 32, TI = 32, TV = 4, BLOCK = 256, NTR = 1, ESZ = 2, RED = 1, NBUF = 1, PERSIST = 0 }; static constexpr unsigned long long NT = 0ull;
  static constexpr int mode(int i) { constexpr int m[] = {2, 0, 0}; return m[i]; }
  static constexpr int slot(int i) { constexpr int m[] = {0, -1, -1}; return m[i]; } };
extern "C" __global__ __launch_bounds__(256) void check_tr_red(thx::EwTrParams<3, 3, int> p, thx::EwRedParams<2, 1> q) { thx::ew_tr_red_body<CheckFR, PlanTrRed>(p, q); }
extern "C" __global__ __launch_bounds__(256) void check_tr(thx::EwTrParams<3, 3, int> p, unsigned total) { thx::ew_tr_body<CheckF, PlanTr>(p, total); }
extern "C" __global__ __launch_bounds__(256) void check_ew1(thx::EwParams<3, 1, int> p) { thx::ew_body<CheckF, PlanEw1>(p); }
extern "C" __global__ __launch_bounds__(256) void check_ew3(thx::EwParams<3, 3, long long> p) { thx::ew_body<CheckF, PlanEw3>(p); }
extern "C" __global__ __launch_bounds__(256) void check_row(thx::RowParams<1, 2, 1, 2, int> p) { thx::red_row_body<CheckR, PlanRow>(p); }
extern "C" __global__ __launch_bounds__(256) void check_rows(thx::RowParams<1, 2, 1, 1, int> p) { thx::red_row_body<CheckR, PlanRowS>(p); }
extern "C" __global__ __launch_bounds__(256) void check_col(thx::ColParams<1, 2, 1, 1, int> p) { thx::red_col_body<CheckR, PlanCol>(p); }
extern "C" __global__ __launch_bounds__(256) void check_strip(thx::StripParams<1, 2, 1> p) { thx::red_strip_body<CheckR, PlanStrip>(p); }
extern "C" __global__ __launch_bounds__(256) void check_gen(thx::GenParams<1, 2, 1, 3, 3, int> p) { thx::red_gen_body<CheckR, PlanGen>(p); }
extern "C" __global__ __launch_bounds__(256) void check_fin(thx::FinalParams<2, 1> p) { thx::red_final_body<CheckR, 256, 64>(p); }
