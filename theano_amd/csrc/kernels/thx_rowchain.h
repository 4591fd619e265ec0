// Row chains: a whole island of elementwise operations and reductions along
// the last axis (softmax, its gradient, layer-norm style statistics, ...) in
// one kernel. TPR threads own one row and keep it in registers from the first
// load to the last store, so every operand crosses HBM once whatever the
// number of graph nodes in the island.
//
// A generated functor C supplies
//   enum { NIN, NOUT };
//   template <class X> static void row(X& x);   // the island, straight-line
// written against the context X below: loads and stores of full rows
// (per-element values live in T v[X::NCH][X::VEC]), of per-row and per-column
// operands, and all-lane reductions.
#pragma once

namespace thx {

template <int NIN, int NOUT, class IT>
struct RowChainParams {
  char* in[NIN];
  unsigned long long imm[NIN];   // value of host scalars
  char* out[NOUT];
  long long rows;
  int cols;                      // row length C
  int cv;                        // C / VEC
  IT in_rstride[NIN];            // elements between consecutive rows (0 for per-column operands)
  IT out_rstride[NOUT];
};

// Plan members: typedef IT; enum { VEC, NCH, TPR, BLOCK }; static constexpr unsigned long long NT, NTO (bit i:
// input / output i is accessed non-temporally); static constexpr int imm(int input).
template <class C, class P>
struct RowCtx {
  typedef typename P::IT IT;
  enum { VEC = P::VEC, NCH = P::NCH, TPR = P::TPR };
  const RowChainParams<C::NIN, C::NOUT, IT>& p;
  long long row;
  int lane;
  bool live;

  THX_DEV RowCtx(const RowChainParams<C::NIN, C::NOUT, IT>& p_) : p(p_) {
    row = (long long)blockIdx.x * (P::BLOCK / TPR) + threadIdx.x / TPR;
    lane = threadIdx.x % TPR;
    live = row < p.rows;
    if (!live) row = 0;
  }
  THX_DEV bool valid(int ch) const { return ch * TPR + lane < p.cv; }

  // a full operand: one element per (row, column)
  template <int I, class T, class CT>
  THX_DEV void load_full(CT (&v)[NCH][VEC]) const {
    const T* base = (const T*)p.in[I] + (IT)row * p.in_rstride[I];
#pragma unroll
    for (int ch = 0; ch < NCH; ++ch) {
      Vec<T, VEC> r;
#pragma unroll
      for (int k = 0; k < VEC; ++k) r.v[k] = T();
      if (valid(ch)) load_vec<T, VEC, ((P::NT >> I) & 1) != 0>(r, base + (IT)(ch * TPR + lane) * VEC);
#pragma unroll
      for (int k = 0; k < VEC; ++k) v[ch][k] = (CT)r.v[k];
    }
  }
  // a per-column operand shared by all rows (row stride 0): same code path
  template <int I, class T, class CT>
  THX_DEV void load_col(CT (&v)[NCH][VEC]) const {
    load_full<I, T, CT>(v);
  }
  // one value per row
  template <int I, class T, class CT>
  THX_DEV void load_row(CT& s) const {
    s = (CT)((const T*)p.in[I])[(IT)row * p.in_rstride[I]];
  }
  // one value for the whole launch: a host scalar in the arguments or a device scalar
  template <int I, class T, class CT>
  THX_DEV void load_scalar(CT& s) const {
    if (P::imm(I)) s = (CT) * (const T*)&p.imm[I];
    else s = (CT) * (const T*)p.in[I];
  }
  template <int O, class T, class CT>
  THX_DEV void store_full(const CT (&v)[NCH][VEC]) const {
    T* base = (T*)p.out[O] + (IT)row * p.out_rstride[O];
#pragma unroll
    for (int ch = 0; ch < NCH; ++ch) {
      Vec<T, VEC> r;
#pragma unroll
      for (int k = 0; k < VEC; ++k) r.v[k] = (T)v[ch][k];
      if (live && valid(ch)) store_vec<T, VEC, ((P::NTO >> O) & 1) != 0>(base + (IT)(ch * TPR + lane) * VEC, r);
    }
  }
  template <int O, class T, class CT>
  THX_DEV void store_row(const CT s) const {
    if (live && lane == 0) ((T*)p.out[O])[(IT)row * p.out_rstride[O]] = (T)s;
  }

  // combine one value per lane across the TPR lanes of the row; every lane
  // gets the result. Op::comb(a, b) folds b into a.
  template <class Op, class A>
  THX_DEV A allreduce(A a) const {
    if (TPR <= THX_WAVE) {
#pragma unroll
      for (int m = TPR / 2; m >= 1; m >>= 1) {
        A b = shfl_xor_t(a, m);
        Op::comb(a, b);
      }
      return a;
    } else {
      __shared__ A lds[P::BLOCK / THX_WAVE];
#pragma unroll
      for (int m = THX_WAVE / 2; m >= 1; m >>= 1) {
        A b = shfl_xor_t(a, m);
        Op::comb(a, b);
      }
      __syncthreads();
      if ((threadIdx.x & (THX_WAVE - 1)) == 0) lds[threadIdx.x / THX_WAVE] = a;
      __syncthreads();
      A r = lds[0];
#pragma unroll
      for (int w = 1; w < P::BLOCK / THX_WAVE; ++w) Op::comb(r, lds[w]);
      return r;
    }
  }
};

template <class C, class P>
__device__ __forceinline__ void rowchain_body(const RowChainParams<C::NIN, C::NOUT, typename P::IT>& p) {
  RowCtx<C, P> x(p);
  C::row(x);
}

}  // namespace thx
