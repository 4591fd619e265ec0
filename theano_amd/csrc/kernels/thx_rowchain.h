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
  int cv;                        // vectors in a row: C / VEC, rounded up when the plan has UA
  IT in_rstride[NIN];            // elements between consecutive rows (0 for per-column operands)
  IT out_rstride[NOUT];
};

// Plan members: typedef IT; enum { VEC, NCH, TPR, BLOCK, UA }; static constexpr unsigned long long NT, NTO (bit i:
// input / output i is accessed non-temporally); static constexpr int imm(int input).
// UA: rows that do not start on vector boundaries or are no whole number of vectors long (1001 classes): vectors go
// through element-aligned pointers, and the last vector of a row ends with the row and overlaps the one before it -
// the elements it repeats are computed and stored twice (same values) and left out of reductions (`counts`).
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
  // first element of the vector (ch, lane) in its row
  THX_DEV IT first(int ch) const {
    const int q = ch * TPR + lane;
    if (P::UA != 0 && q == p.cv - 1) return (IT)(p.cols - VEC);
    return (IT)q * VEC;
  }
  // does element k of vector ch take part in reductions (it does not when the row's last vector repeats it)
  THX_DEV bool counts(int ch, int k) const {
    if (P::UA == 0) return true;
    return !(ch * TPR + lane == p.cv - 1 && k < p.cv * VEC - p.cols);
  }

  // a full operand: one element per (row, column)
  template <int I, class T, class CT>
  THX_DEV void load_full(CT (&v)[NCH][VEC]) const {
    const T* base = (const T*)p.in[I] + (IT)row * p.in_rstride[I];
#pragma unroll
    for (int ch = 0; ch < NCH; ++ch) {
      Vec<T, VEC> r;
#pragma unroll
      for (int k = 0; k < VEC; ++k) r.v[k] = T();
      if (valid(ch)) load_vec<T, VEC, ((P::NT >> I) & 1) != 0, P::UA != 0>(r, base + first(ch));
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
      if (live && valid(ch)) store_vec<T, VEC, ((P::NTO >> O) & 1) != 0, P::UA != 0>(base + first(ch), r);
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

// ---------------------------------------------------------------------------
// "Held" form: the reduce domain of one kept index k is RA slabs of RC
// contiguous elements (sum over axes (0, 2, 3) of an [N, C, H, W] array keeps
// k = c: RA = N slabs of RC = H * W elements; a plain long row is RA = 1).
// One block owns one k and keeps every full-shaped input of the island on chip
// in its storage type - packed in registers, the rest in LDS - from the one
// load to the last store, however many reductions and elementwise steps lie
// between: a (256, 256, 28, 28) float16 batch normalisation reads x once and
// writes y once, with mean and variance taken in two true passes over the
// held values.
//
// The generated functor supplies
//   template <class X> static void held(X& x);
// in which per-element values are never stored: every loop over the held
// chunks (one per group of reductions, one for the stores) recomputes the
// elementwise steps it needs from the raw inputs and the per-k scalars.
template <int NIN, int NOUT, class IT>
struct HeldParams {
  char* in[NIN];
  unsigned long long imm[NIN];   // value of host scalars
  char* out[NOUT];
  IT in_sa[NIN], in_sk[NIN];     // bytes between slabs, bytes between kept indices
  IT out_sa[NOUT], out_sk[NOUT];
  FastDiv bvfd;                  // RC / VEC
  unsigned nvec;                 // vectors per kept index: RA * RC / VEC
  unsigned bv;                   // RC / VEC
  unsigned dra, dcv;             // BLOCK / bv, BLOCK % bv: how (slab, vector) advance from one chunk to the next
};

// Plan members: typedef IT (unsigned: every byte offset fits 32 bits; long long otherwise);
// enum { VEC, NCH, NFULL (chunks that every thread of the block has), BLOCK, LDS_BYTES };
// static constexpr unsigned long long NT, NTO;
// static constexpr int imm(int input), nlds(int input) (leading chunks of that input kept in LDS),
// ldsoff(int input) (where they start).
template <class C, class P>
struct HeldCtx {
  typedef typename P::IT IT;
  enum { VEC = P::VEC, NCH = P::NCH, BLOCK = P::BLOCK };
  const HeldParams<C::NIN, C::NOUT, IT>& p;
  unsigned char* stash;
  unsigned k, t;

  THX_DEV HeldCtx(const HeldParams<C::NIN, C::NOUT, IT>& p_, unsigned char* s) : p(p_), stash(s) {
    // Consecutive blocks go to the eight dies in turn, each with its own L2.  Neighbouring kept indices
    // share cache lines where their slabs meet (a 1568-byte slab ends inside a 128-byte line), so each die
    // takes one contiguous eighth of the indices and those lines are fetched once.
    const unsigned b = blockIdx.x, nb = gridDim.x;
    k = (nb & 7) == 0 ? (b & 7) * (nb >> 3) + (b >> 3) : b;
    t = threadIdx.x;
  }
  // chunks below NFULL are inside the reduce domain for every thread
  THX_DEV bool valid(int ch) const { return ch < P::NFULL || (unsigned)ch * BLOCK + t < p.nvec; }
  // End of one chunk in a loop over the held values: nothing moves across it.  Left alone, the
  // scheduler interleaves many chunks (and hoists the LDS reads of all of them) for parallelism the
  // four waves of a SIMD already provide, and the registers that takes push held values out to memory.
  THX_DEV static void pace(int) { __builtin_amdgcn_sched_barrier(0); }
  // An accumulator at the end of a chunk: its value exists here, so the arithmetic that feeds it cannot
  // drift below the loads of the chunks that follow (which would keep all their data alive).
  template <class A>
  THX_DEV static void pin(A& a) {
    if constexpr (sizeof(A) == 4 || sizeof(A) == 8) {
      if constexpr (__is_trivially_copyable(A) && !__is_class(A)) asm volatile("" : "+v"(a));
    }
  }

  // (slab, vector inside the slab) of this thread's chunk; recomputed by every loop that needs
  // addresses, through an opaque copy so that the compiler does not keep NCH offsets alive instead
  struct Pos { unsigned ra, cv; };
  THX_DEV Pos begin() const {
    Pos q;
    divmod(t, p.bvfd, q.ra, q.cv);
    asm volatile("" : "+v"(q.ra), "+v"(q.cv));
    return q;
  }
  THX_DEV void next(Pos& q) const {
    q.ra += p.dra;
    q.cv += p.dcv;
    if (q.cv >= p.bv) {
      q.cv -= p.bv;
      q.ra += 1;
    }
  }

  template <int I, class T>
  struct Held {
    enum { BYTES = VEC * (int)sizeof(T), WORDS = (BYTES + 3) / 4, NL = P::nlds(I), NR = NCH - NL };
    unsigned w[NR > 0 ? NR : 1][WORDS];
  };
  template <int I, class T>
  THX_DEV void hold(Held<I, T>& h) const {
    typedef Held<I, T> H;
    const char* base = p.in[I] + (IT)k * p.in_sk[I];
    Pos q = begin();
    if (H::NL > 0) {
      // the chunks that live in LDS come first: their registers are free again before the rest is in flight
      Vec<T, VEC> tmp[H::NL > 0 ? H::NL : 1];
#pragma unroll
      for (int ch = 0; ch < H::NL; ++ch) {
#pragma unroll
        for (int j = 0; j < VEC; ++j) tmp[ch].v[j] = T();
        if (valid(ch)) load_vec<T, VEC, ((P::NT >> I) & 1) != 0>(tmp[ch], (const T*)(base + (IT)q.ra * p.in_sa[I] + (IT)q.cv * H::BYTES));
        next(q);
      }
#pragma unroll
      for (int ch = 0; ch < H::NL; ++ch)
        *(Vec<T, VEC>*)(stash + P::ldsoff(I) + ((unsigned)ch * BLOCK + t) * H::BYTES) = tmp[ch];
      __builtin_amdgcn_sched_barrier(0);
    }
#pragma unroll
    for (int ch = H::NL; ch < NCH; ++ch) {
      Vec<T, VEC> r;
#pragma unroll
      for (int j = 0; j < VEC; ++j) r.v[j] = T();
      if (valid(ch)) load_vec<T, VEC, ((P::NT >> I) & 1) != 0>(r, (const T*)(base + (IT)q.ra * p.in_sa[I] + (IT)q.cv * H::BYTES));
#pragma unroll
      for (int j = 0; j < H::WORDS; ++j) h.w[ch - H::NL][j] = 0;
      __builtin_memcpy(&h.w[ch - H::NL][0], &r, H::BYTES);
      next(q);
    }
  }
  template <int I, class T>
  THX_DEV Vec<T, VEC> get(const Held<I, T>& h, int ch) const {
    typedef Held<I, T> H;
    Vec<T, VEC> r;
    if (ch < H::NL) r = *(const Vec<T, VEC>*)(stash + P::ldsoff(I) + ((unsigned)ch * BLOCK + t) * H::BYTES);
    else __builtin_memcpy(&r, &h.w[ch >= H::NL ? ch - H::NL : 0][0], H::BYTES);
    return r;
  }
  // Between two loops over the held values: what one loop derived from them (conversions to the
  // compute type) must not stay in registers for the next one.
  template <int I, class T>
  THX_DEV void fence(Held<I, T>& h) const {
    typedef Held<I, T> H;
#pragma unroll
    for (int c = 0; c < H::NR; ++c) {
#pragma unroll
      for (int j = 0; j < H::WORDS; ++j) asm volatile("" : "+v"(h.w[c][j]));
    }
  }
  template <int O, class T>
  THX_DEV void put(const Pos& q, const Vec<T, VEC>& v) const {
    char* base = p.out[O] + (IT)k * p.out_sk[O];
    store_vec<T, VEC, ((P::NTO >> O) & 1) != 0>((T*)(base + (IT)q.ra * p.out_sa[O] + (IT)q.cv * (VEC * (int)sizeof(T))), v);
  }
  // A value that is the same in every lane moves to scalar registers: a chain carries a dozen or more
  // per-index values through its loops, and the vector registers are for the held elements.
  template <class CT>
  THX_DEV static CT uni(CT v) {
    if constexpr (sizeof(CT) == 4) {
      return __builtin_bit_cast(CT, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, v)));
    } else if constexpr (sizeof(CT) == 8) {
      const unsigned long long b = __builtin_bit_cast(unsigned long long, v);
      const unsigned lo = (unsigned)__builtin_amdgcn_readfirstlane((int)(unsigned)b);
      const unsigned hi = (unsigned)__builtin_amdgcn_readfirstlane((int)(unsigned)(b >> 32));
      return __builtin_bit_cast(CT, ((unsigned long long)hi << 32) | lo);
    } else if constexpr (sizeof(CT) < 4) {
      return (CT)__builtin_amdgcn_readfirstlane((int)v);
    } else {
      return v;
    }
  }
  template <int I, class T, class CT>
  THX_DEV void load_row(CT& s) const {
    s = (CT) * (const T*)(p.in[I] + (IT)k * p.in_sk[I]);
  }
  template <int I, class T, class CT>
  THX_DEV void load_scalar(CT& s) const {
    if (P::imm(I)) s = (CT) * (const T*)&p.imm[I];
    else s = (CT) * (const T*)p.in[I];
  }
  template <int O, class T, class CT>
  THX_DEV void store_row(const CT s) const {
    if (t == 0) *(T*)(p.out[O] + (IT)k * p.out_sk[O]) = (T)s;
  }
  // Every lane gets the combination over the block.  The partial results of the waves are folded by a
  // second butterfly over one value per lane (reading all of them into every thread would take
  // two registers per wave and value, which the held values need).
  template <class Op, class A>
  THX_DEV A allreduce(A a) const {
    constexpr int NW = BLOCK / THX_WAVE;
    __shared__ A lds[NW];
#pragma unroll
    for (int m = THX_WAVE / 2; m >= 1; m >>= 1) {
      A b = shfl_xor_t(a, m);
      Op::comb(a, b);
    }
    if (NW == 1) return a;          // a block of one wave: the butterfly was all of it
    __syncthreads();
    if ((t & (THX_WAVE - 1)) == 0) lds[t / THX_WAVE] = a;
    __syncthreads();
    A r = lds[t & (NW - 1)];
#pragma unroll
    for (int m = NW / 2; m >= 1; m >>= 1) {
      A b = shfl_xor_t(r, m);
      Op::comb(r, b);
    }
    return r;
  }
};

template <class C, class P>
__device__ __forceinline__ void heldchain_body(const HeldParams<C::NIN, C::NOUT, typename P::IT>& p) {
  __shared__ __attribute__((aligned(16))) unsigned char stash[P::LDS_BYTES > 0 ? P::LDS_BYTES : 16];
  HeldCtx<C, P> x(p, stash);
  C::held(x);
}

}  // namespace thx
