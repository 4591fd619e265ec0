// N-ary strided/broadcast elementwise kernels.
//
// A generated functor F supplies
//   enum { NIN, NOUT, NOPS = NIN + NOUT };
//   template <int V> struct Regs;                       // one Vec per operand
//   template <int V, class A> static void load(const A&, Regs<V>&);
//   template <int V> static void compute(Regs<V>&);     // the scalar graph, V times
//   template <int V, class A> static void store(const A&, const Regs<V>&);
// and a generated plan P supplies
//   typedef int|long long IT;  enum { ND, VEC, UNR, BLOCK, GS (grid-stride loop over chunks),
//     UA (vectors through element-aligned pointers), RAG (ND > 1: the rows are no whole number of vectors; the
//     last vector of a row holds fd[ND - 1].pad elements and is handled element by element) };
//   static constexpr unsigned long long NT;             // bit i: operand i is accessed non-temporally
//   static constexpr int mode(int operand);             // M_VEC / M_BCAST / M_GATHER
//   static constexpr int sclass(int operand, int dim);  // stride is 0 / is 1 / anything (2)
//   static constexpr int alias(int operand);            // first operand with identical strides
// The host collapses dimensions, so ND is the rank after merging every pair of
// neighbouring dimensions that all operands walk with compatible strides.
#pragma once

namespace thx {

template <int NOPS, int ND, class IT>
struct EwParams {
  char* ptr[NOPS];       // operand base addresses (inputs, then outputs)
  unsigned long long imm[NOPS];  // value bytes of M_IMM operands
  long long nvec;        // whole vectors to process
  long long n;           // elements in total
  FastDiv fd[ND];        // extent of each dimension; the last one counts vectors
  IT stride[NOPS][ND];   // element strides, 0 where an operand broadcasts
};

template <class P, int NOPS>
struct EwAcc {
  typedef typename P::IT IT;
  char* const* ptr;
  const unsigned long long* imm;
  const IT (*stride)[P::ND];
  IT off[NOPS];
  bool last;             // RAG: this is the last vector of its row

  template <int I, class T, int N>
  THX_DEV void ld(Vec<T, N>& r) const {
    if (P::mode(I) == M_IMM) {
      const T s = *(const T*)&imm[I];
#pragma unroll
      for (int k = 0; k < N; ++k) r.v[k] = s;
      return;
    }
    const T* b = (const T*)ptr[I] + off[I];
    if (N == 1) {
      r.v[0] = *b;
    } else if (P::mode(I) == M_VEC) {
      load_vec<T, N, ((P::NT >> I) & 1) != 0, P::UA != 0>(r, b);
    } else if (P::mode(I) == M_BCAST) {
      const T s = *b;
#pragma unroll
      for (int k = 0; k < N; ++k) r.v[k] = s;
    } else {
      const IT st = stride[I][P::ND - 1];
#pragma unroll
      for (int k = 0; k < N; ++k) r.v[k] = b[k * st];
    }
  }

  template <int I, class T, int N>
  THX_DEV void st(const Vec<T, N>& r) const {
    T* b = (T*)ptr[I] + off[I];
    if (N == 1) {
      *b = r.v[0];
    } else if (P::mode(I) == M_VEC) {
      store_vec<T, N, ((P::NT >> I) & 1) != 0, P::UA != 0>(b, r);
    } else {
      const IT st = stride[I][P::ND - 1];
#pragma unroll
      for (int k = 0; k < N; ++k) b[k * st] = r.v[k];
    }
  }
};

// coordinate * stride with the multiply only where the plan could not rule it out
template <class P, class IT>
THX_DEV IT ew_term(int operand, int dim, IT coord, IT stride) {
  return P::sclass(operand, dim) == 0 ? (IT)0 : (P::sclass(operand, dim) == 1 ? coord : coord * stride);
}

// One thread handles UNR vectors, BLOCK apart, so a wave's accesses stay
// contiguous; all loads are issued before any arithmetic or store.
template <class F, class P>
__device__ __forceinline__ void ew_body(const EwParams<F::NOPS, P::ND, typename P::IT>& p) {
  typedef typename P::IT IT;
  typedef typename UnsignedOf<IT>::type UT;
  constexpr int VEC = P::VEC, UNR = P::UNR, ND = P::ND, NOPS = F::NOPS;

  const long long step = P::GS ? (long long)gridDim.x * (P::BLOCK * UNR) : p.nvec + 1;
  for (long long q0 = (long long)blockIdx.x * (P::BLOCK * UNR) + threadIdx.x;
       q0 - threadIdx.x < p.nvec; q0 += step) {
  typename F::template Regs<VEC> r[UNR];
  EwAcc<P, NOPS> a[UNR];
  bool full[UNR];
#pragma unroll
  for (int u = 0; u < UNR; ++u) {
    const long long q = q0 + (long long)u * P::BLOCK;
    full[u] = q < p.nvec;
    a[u].ptr = p.ptr;
    a[u].imm = p.imm;
    a[u].stride = p.stride;
    // offset of the vector in every operand: sum over dimensions of coordinate * stride, where the
    // plan says which strides are 0 or 1 (no multiply; 32-bit integer multiplies run at quarter
    // rate) and which operands walk memory exactly like an earlier one (same offset)
    if (ND == 1) {
#pragma unroll
      for (int i = 0; i < NOPS; ++i) a[u].off[i] = ew_term<P>(i, 0, (IT)(q * VEC), p.stride[i][0]);
    } else {
      UT rem = (UT)(full[u] ? q : 0), c;
      divmod(rem, p.fd[ND - 1], rem, c);
      a[u].last = c + 1 == p.fd[ND - 1].d;
#pragma unroll
      for (int i = 0; i < NOPS; ++i)
        if (P::alias(i) == i) a[u].off[i] = ew_term<P>(i, ND - 1, (IT)(c * VEC), p.stride[i][ND - 1]);
#pragma unroll
      for (int d = ND - 2; d >= 1; --d) {
        divmod(rem, p.fd[d], rem, c);
#pragma unroll
        for (int i = 0; i < NOPS; ++i)
          if (P::alias(i) == i) a[u].off[i] += ew_term<P>(i, d, (IT)c, p.stride[i][d]);
      }
#pragma unroll
      for (int i = 0; i < NOPS; ++i)
        if (P::alias(i) == i) a[u].off[i] += ew_term<P>(i, 0, (IT)rem, p.stride[i][0]);
#pragma unroll
      for (int i = 0; i < NOPS; ++i)
        if (P::alias(i) != i) a[u].off[i] = a[u].off[P::alias(i)];
    }
    if constexpr (P::RAG != 0 && ND > 1) {
      const int mine = (int)p.fd[ND - 1].pad;
      if (full[u] && mine < VEC && a[u].last) {
        for (int k = 0; k < mine; ++k) {
          typename F::template Regs<1> r1;
          EwAcc<P, NOPS> a1 = a[u];
#pragma unroll
          for (int i = 0; i < NOPS; ++i) a1.off[i] = a[u].off[i] + ew_term<P>(i, ND - 1, (IT)k, p.stride[i][ND - 1]);
          F::template load<1>(a1, r1);
          F::template compute<1>(r1);
          F::template store<1>(a1, r1);
        }
        full[u] = false;
      }
    }
    if (full[u]) F::template load<VEC>(a[u], r[u]);
  }
#pragma unroll
  for (int u = 0; u < UNR; ++u)
    if (full[u]) F::template compute<VEC>(r[u]);
#pragma unroll
  for (int u = 0; u < UNR; ++u)
    if (full[u]) F::template store<VEC>(a[u], r[u]);
  }

  // ND == 1 only: the elements after the last whole vector, one per thread.
  if (ND == 1 && VEC > 1) {
    const long long tail0 = (p.n / VEC) * VEC;
    const long long e = tail0 + threadIdx.x;
    if (blockIdx.x == 0 && e < p.n) {
      typename F::template Regs<1> r1;
      EwAcc<P, NOPS> a1;
      a1.ptr = p.ptr;
      a1.imm = p.imm;
      a1.stride = p.stride;
#pragma unroll
      for (int i = 0; i < NOPS; ++i) a1.off[i] = (IT)e * p.stride[i][0];
      F::template load<1>(a1, r1);
      F::template compute<1>(r1);
      F::template store<1>(a1, r1);
    }
  }
}

// ---------------------------------------------------------------------------
// Permuted-read variant. Some inputs are unit-stride along a dimension T that
// is not the innermost one of the result (a dimshuffled view). A block owns a
// TT x TI patch of (T, innermost): those inputs are read in rows of TT elements
// along T - whole cache lines - into LDS and read back transposed, while every
// other operand is accessed along the innermost dimension. Rows of a tile are
// padded by one element so that the transposed reads hit distinct banks.
//
// Extra plan members: enum { TT, TI, TV (elements per access), NTR (staged
// inputs), ESZ (largest staged element) }; static constexpr int slot(int
// operand): LDS slot or -1.
//
// With plan member RED = 1 the kernel also reduces results over every dimension but the innermost
// (the per-channel sum of an NHWC result that is written anyway): the functor names a reduction
// functor `Red` (contract in thx_reduce.h) and feeds it element k of a thread's results through
// `red_lane`.  A block then walks `rowtiles / groups` tiles of one and the same innermost range,
// keeps TV accumulators per thread across them, merges the rows of its tile shape through LDS
// and leaves one partial per innermost index, laid out [group][index] for the reductions' final
// pass (or the result itself when there is one group).
template <int NOPS, int ND, class IT>
struct EwTrParams {
  char* ptr[NOPS];
  unsigned long long imm[NOPS];
  int ext_t, ext_i;         // extents of dimension T and of the innermost dimension
  FastDiv tiles_i, tiles_t;  // tiles along each of them
  FastDiv ofd[ND];          // extents of the other (outer) dimensions, ND - 2 of them used
  IT ostride[NOPS][ND];     // strides along the outer dimensions
  IT tstride[NOPS];
  IT istride[NOPS];
};

// What the reducing variant needs beyond EwTrParams.
template <int NOUT, int NEX>
struct EwRedParams {
  RedOut<NOUT, NEX> out;    // results of the reduction (one element per innermost index)
  char* partial;            // Acc[groups][ext_i] when groups > 1
  int rowtiles;             // tiles over all dimensions but the innermost one
  int groups;               // blocks that share one innermost range
};

template <class P, int NOPS>
struct TrStageAcc {  // global -> LDS for the staged inputs, nothing for the others
  typedef typename P::IT IT;
  char* const* ptr;
  unsigned char* lds;
  IT off[NOPS];
  int cell;  // LDS index of the first element: row * (TT + 1) + position along T
  template <int I, class T, int N>
  THX_DEV void ld(Vec<T, N>&) const {
    if (P::slot(I) >= 0) {
      T* tile = (T*)(lds + P::slot(I) * (P::TI * (P::TT + 1) * P::ESZ));
      Vec<T, N> r;
      load_vec<T, N, ((P::NT >> I) & 1) != 0>(r, (const T*)ptr[I] + off[I]);
#pragma unroll
      for (int k = 0; k < N; ++k) tile[cell + k] = r.v[k];
    }
  }
};

template <class P, int NOPS>
struct TrFetchAcc {  // global -> registers for the staged inputs, nothing for the others
  typedef typename P::IT IT;
  char* const* ptr;
  IT off[NOPS];
  template <int I, class T, int N>
  THX_DEV void ld(Vec<T, N>& r) const {
    if (P::slot(I) >= 0) load_vec<T, N, ((P::NT >> I) & 1) != 0>(r, (const T*)ptr[I] + off[I]);
  }
};

template <class P, int NOPS>
struct TrPutAcc {  // registers -> LDS for the staged inputs (visits the operands like a load)
  unsigned char* lds;
  int cell;  // LDS index of the first element: row * (TT + 1) + position along T
  template <int I, class T, int N>
  THX_DEV void ld(Vec<T, N>& r) const {
    if (P::slot(I) >= 0) {
      T* tile = (T*)(lds + P::slot(I) * (P::TI * (P::TT + 1) * P::ESZ));
#pragma unroll
      for (int k = 0; k < N; ++k) tile[cell + k] = r.v[k];
    }
  }
};

template <class P, int NOPS>
struct TrAcc {  // LDS (transposed) or global -> registers, registers -> global
  typedef typename P::IT IT;
  char* const* ptr;
  const unsigned long long* imm;
  const unsigned char* lds;
  IT off[NOPS];
  int cell;  // LDS index of the first element: position along the inner dimension * (TT + 1) + row along T
  template <int I, class T, int N>
  THX_DEV void ld(Vec<T, N>& r) const {
    if (P::slot(I) >= 0) {
      const T* tile = (const T*)(lds + P::slot(I) * (P::TI * (P::TT + 1) * P::ESZ));
#pragma unroll
      for (int k = 0; k < N; ++k) r.v[k] = tile[cell + k * (P::TT + 1)];
    } else if (P::mode(I) == M_IMM) {
      const T s = *(const T*)&imm[I];
#pragma unroll
      for (int k = 0; k < N; ++k) r.v[k] = s;
    } else if (P::mode(I) == M_BCAST) {
      const T s = *((const T*)ptr[I] + off[I]);
#pragma unroll
      for (int k = 0; k < N; ++k) r.v[k] = s;
    } else {
      load_vec<T, N, ((P::NT >> I) & 1) != 0>(r, (const T*)ptr[I] + off[I]);
    }
  }
  template <int I, class T, int N>
  THX_DEV void st(const Vec<T, N>& r) const {
    store_vec<T, N, ((P::NT >> I) & 1) != 0>((T*)ptr[I] + off[I], r);
  }
};

// TV consecutive elements per access: along T while staging, along the inner
// dimension while computing. The host guarantees that both extents are
// multiples of TV and that every vector access is aligned.
template <class F, class P>
struct EwTrTile {
  typedef typename P::IT IT;
  static constexpr int TT = P::TT, TI = P::TI, TV = P::TV, NOPS = F::NOPS, ND = P::ND;
  static constexpr int LPR_S = TT / TV;              // staging: lanes per row along T
  static constexpr int RPP_S = P::BLOCK / LPR_S;     //          rows (positions along the inner dimension) per pass
  static constexpr int PASSES_S = TI / RPP_S;
  static constexpr int LPR_C = TI / TV;              // computing: lanes per row along the inner dimension
  static constexpr int RPP_C = P::BLOCK / LPR_C;     //            rows (positions along T) per pass
  static constexpr int PASSES_C = TT / RPP_C;
  static constexpr int UNR = PASSES_C < 4 ? PASSES_C : 4;
  static constexpr int LDS_BYTES = P::NTR * TI * (TT + 1) * P::ESZ;
  static_assert(PASSES_S >= 1 && PASSES_C >= 1 && PASSES_S * RPP_S == TI && PASSES_C * RPP_C == TT,
                "tile and block do not divide");

  // Where tile `rem` (counted over the dimensions other than the innermost) starts: element offsets of
  // every operand without the tile's own two dimensions, and its first position along T.
  static __device__ __forceinline__ void locate(const EwTrParams<NOPS, ND, IT>& p, unsigned rem, IT (&base)[NOPS], int& t0) {
    unsigned tt, c;
    divmod(rem, p.tiles_t, rem, tt);
#pragma unroll
    for (int i = 0; i < NOPS; ++i) base[i] = 0;
#pragma unroll
    for (int d = ND - 3; d >= 1; --d) {
      divmod(rem, p.ofd[d], rem, c);
#pragma unroll
      for (int i = 0; i < NOPS; ++i) base[i] += (IT)c * p.ostride[i][d];
    }
    if (ND >= 3) {
#pragma unroll
      for (int i = 0; i < NOPS; ++i) base[i] += (IT)rem * p.ostride[i][0];
    }
    t0 = tt * TT;
  }

  typedef typename F::template Regs<TV> Regs;

  // stage, first half: the staged inputs of one tile from memory into registers (lanes run along T)
  static __device__ __forceinline__ void fetch(const EwTrParams<NOPS, ND, IT>& p, const IT (&base)[NOPS], int t0, int i0,
                                               Regs (&s)[PASSES_S]) {
    const int lane = threadIdx.x % LPR_S, row = threadIdx.x / LPR_S;
    const int t = t0 + lane * TV;
#pragma unroll
    for (int k = 0; k < PASSES_S; ++k) {
      const int i = i0 + row + k * RPP_S;
      if (t < p.ext_t && i < p.ext_i) {
        TrFetchAcc<P, NOPS> a;
        a.ptr = p.ptr;
#pragma unroll
        for (int o = 0; o < NOPS; ++o) a.off[o] = base[o] + (IT)t * p.tstride[o] + (IT)i * p.istride[o];
        F::template load<TV>(a, s[k]);
      }
    }
  }
  // stage, second half: registers into the LDS tile
  static __device__ __forceinline__ void put(const EwTrParams<NOPS, ND, IT>& p, unsigned char* lds, int t0, int i0,
                                             Regs (&s)[PASSES_S]) {
    const int lane = threadIdx.x % LPR_S, row = threadIdx.x / LPR_S;
    const int t = t0 + lane * TV;
#pragma unroll
    for (int k = 0; k < PASSES_S; ++k) {
      const int ii = row + k * RPP_S;
      if (t < p.ext_t && i0 + ii < p.ext_i) {
        TrPutAcc<P, NOPS> a;
        a.lds = lds;
        a.cell = ii * (TT + 1) + lane * TV;
        F::template load<TV>(a, s[k]);
      }
    }
  }

  // compute: lanes run along the innermost dimension.  ACC: per-thread accumulators of the reducing
  // variant (one per element of a vector), or a dummy.
  template <class ACC>
  static __device__ __forceinline__ void compute(const EwTrParams<NOPS, ND, IT>& p, const unsigned char* lds,
                                                 const IT (&base)[NOPS], int t0, int i0, ACC* acc) {
    const int lane = threadIdx.x % LPR_C, row = threadIdx.x / LPR_C;
    const int i = i0 + lane * TV;
#pragma unroll
    for (int k0 = 0; k0 < PASSES_C; k0 += UNR) {
      Regs r[UNR];
      TrAcc<P, NOPS> a[UNR];
      bool ok[UNR];
#pragma unroll
      for (int u = 0; u < UNR; ++u) {
        const int tl = row + (k0 + u) * RPP_C, t = t0 + tl;
        ok[u] = t < p.ext_t && i < p.ext_i;
        a[u].ptr = p.ptr;
        a[u].imm = p.imm;
        a[u].lds = lds;
        a[u].cell = lane * TV * (TT + 1) + tl;
#pragma unroll
        for (int o = 0; o < NOPS; ++o) a[u].off[o] = base[o] + (IT)t * p.tstride[o] + (IT)i * p.istride[o];
        if (ok[u]) F::template load<TV>(a[u], r[u]);
      }
#pragma unroll
      for (int u = 0; u < UNR; ++u)
        if (ok[u]) F::template compute<TV>(r[u]);
#pragma unroll
      for (int u = 0; u < UNR; ++u)
        if (ok[u]) F::template store<TV>(a[u], r[u]);
      if constexpr (P::RED != 0) {
#pragma unroll
        for (int u = 0; u < UNR; ++u)
          if (ok[u]) F::template red_lanes<TV>(acc, r[u]);
      }
    }
  }

  // Tiles first, first + step, ... below `total`, counted with the innermost dimension fastest.  The next
  // tile's inputs are on their way (memory -> registers) while this one is computed from LDS and stored;
  // with two LDS buffers (P::NBUF) one barrier per tile is enough: a buffer is staged again only after the
  // barrier of the tile in between, which every thread reaches after it has finished reading that buffer.
  template <class ACC>
  static __device__ __forceinline__ void walk(const EwTrParams<NOPS, ND, IT>& p, unsigned char* lds, unsigned first,
                                              unsigned step, unsigned total, ACC* acc) {
    Regs s[PASSES_S];
    IT base[NOPS], nbase[NOPS];
    int t0 = 0, nt0 = 0, i0 = 0, ni0 = 0;
    unsigned id = first;
    if (id < total) {
      unsigned rem, ti;
      divmod(id, p.tiles_i, rem, ti);
      locate(p, rem, base, t0);
      i0 = ti * TI;
      fetch(p, base, t0, i0, s);
    }
    int b = 0;
    while (id < total) {
      unsigned char* buf = lds + b * LDS_BYTES;
      put(p, buf, t0, i0, s);
      __syncthreads();
      const unsigned next = id + step;
      if (next < total) {
        unsigned rem, ti;
        divmod(next, p.tiles_i, rem, ti);
        locate(p, rem, nbase, nt0);
        ni0 = ti * TI;
        fetch(p, nbase, nt0, ni0, s);
      }
      compute(p, buf, base, t0, i0, acc);
      if (P::NBUF == 1) __syncthreads();   // the next tile's staging overwrites what this tile's compute phase read
      else b ^= 1;
#pragma unroll
      for (int o = 0; o < NOPS; ++o) base[o] = nbase[o];
      t0 = nt0;
      i0 = ni0;
      id = next;
    }
  }
};

// One block per tile, or (P::PERSIST) a grid of resident blocks that stride over the tiles.
template <class F, class P>
__device__ __forceinline__ void ew_tr_body(const EwTrParams<F::NOPS, P::ND, typename P::IT>& p, unsigned total) {
  typedef EwTrTile<F, P> Tile;
  __shared__ __attribute__((aligned(16))) unsigned char lds[Tile::LDS_BYTES * P::NBUF];
  Tile::walk(p, lds, blockIdx.x, P::PERSIST ? gridDim.x : total, total, (int*)nullptr);
}

// The reducing variant: block b owns the innermost range b % tiles_i and the tiles g, g + groups, ...
// (g = b / tiles_i) over the other dimensions.
template <class F, class P>
__device__ __forceinline__ void ew_tr_red_body(const EwTrParams<F::NOPS, P::ND, typename P::IT>& p,
                                               const EwRedParams<F::Red::NOUT, F::Red::NEX>& q) {
  typedef EwTrTile<F, P> Tile;
  typedef typename F::Red R;
  typedef typename R::Acc Acc;
  constexpr int TI = P::TI, TV = P::TV, RPP = Tile::RPP_C;
  constexpr int RED_BYTES = RPP * TI * (int)sizeof(Acc);
  __shared__ __attribute__((aligned(16))) unsigned char lds[Tile::LDS_BYTES * P::NBUF > RED_BYTES ? Tile::LDS_BYTES * P::NBUF : RED_BYTES];
  unsigned g = blockIdx.x, ti;
  divmod(g, p.tiles_i, g, ti);
  Acc acc[TV];
#pragma unroll
  for (int k = 0; k < TV; ++k) R::init(acc[k]);
  Tile::walk(p, lds, g * p.tiles_i.d + ti, (unsigned)q.groups * p.tiles_i.d, (unsigned)q.rowtiles * p.tiles_i.d, acc);
  __syncthreads();                // the merge below reuses the tile buffers
  // merge the RPP row lanes of the block: [row][position along the innermost dimension]
  Acc* red = (Acc*)lds;
  const int lane = threadIdx.x % Tile::LPR_C, row = threadIdx.x / Tile::LPR_C;
#pragma unroll
  for (int k = 0; k < TV; ++k) red[row * TI + lane * TV + k] = acc[k];
  __syncthreads();
  if (threadIdx.x < TI) {
    const int i = (int)ti * TI + threadIdx.x;
    if (i < p.ext_i) {
      Acc tot = red[threadIdx.x];
#pragma unroll 4
      for (int y = 1; y < RPP; ++y) R::comb(tot, red[y * TI + threadIdx.x]);
      if (q.groups == 1) {
        R::post(q.out, (long long)i, tot);
      } else {
        ((Acc*)q.partial)[(long long)g * p.ext_i + i] = tot;
      }
    }
  }
}

}  // namespace thx
