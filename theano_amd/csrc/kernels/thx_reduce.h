// Commutative-associative reductions with a fused per-element prologue and a
// fused per-result epilogue.
//
// A generated functor R supplies
//   enum { NIN, NOUT, NEX };                             // NEX further operands feed the epilogue
//   struct Acc;                                          // one field per reduction
//   template <int V> struct Regs;                        // one Vec per input
//   static void init(Acc&);                              // identities
//   template <int V, class A> static void load(const A&, Regs<V>&);
//   template <int V> static void accum(Acc&, const Regs<V>&);        // fold V elements into one Acc
//   template <int V> static void accum_lanes(Acc*, const Regs<V>&);  // element k into acc[k]
//   static void comb(Acc&, const Acc&);                  // merge two partial results
//   static Acc shfl_xor(const Acc&, int mask);
//   template <class O> static void post(const O&, long long index, const Acc&);  // epilogue, casts, stores
// Long reductions are split into S slices whose partial Acc values go to a
// scratch array laid out [slice][output]; a second, small launch (red_final)
// merges them in slice order, so results are reproducible run to run. (Merging
// inside the first launch by the last block to arrive was measured slower on
// gfx950: the device-scope release each block needs costs more than a launch.)
//
// Functors whose accumulators are all boolean (any / all) may instead supply
//   static unsigned long long ticket_pack(const Acc&);   // one count per accumulator, 16 bits each
//   static Acc ticket_unpack(unsigned long long);
// and plans with TICKET = 1 then finish in the first launch: every slice adds its packed flags plus
// 1 << 48 to ONE 64-bit word per output with a single atomic add.  That word is the only object
// shared between the slices, so the atomic operation's own total order decides everything: the
// slice that reads S - 1 in the count field has, in the value the add returned, the contributions of
// all the others, writes the result and puts the word back to zero for the next launch.  No fence,
// no partials, no second launch; counts of true / false flags are order-free, so the result is
// reproducible.
#pragma once

namespace thx {

// Where results go, plus the epilogue's further operands: the value of a host scalar, or the
// address of a device array that holds one element per result, `exs` elements apart (1 for a
// contiguous array; a view such as x[0, :, 0, 0] has the stride of the axis it keeps).
template <int NOUT, int NEX>
struct RedOut {
  char* ptr[NOUT];
  unsigned long long ex[NEX > 0 ? NEX : 1];
  long long exs[NEX > 0 ? NEX : 1];
};

// ---------------------------------------------------------------------------
// "Row" form: every output owns a reduce domain of RA x RC elements, RC being
// the vectorised dimension. TPR threads cooperate on one output; a block holds
// BLOCK / TPR outputs. Covers trailing-axis reductions, whole-array reductions
// (one output, many slices) and outer x kept x inner patterns (RA > 1).
// The slice holding `tot` for output `o` checks in; the last one to do so writes the result.
// `words`: one zero word per output, zero again when the kernel ends.
template <class R, class O>
THX_DEV void ticket_finish(const O& out, unsigned long long* words, long long o, int S, const typename R::Acc& tot) {
  const unsigned long long mine = R::ticket_pack(tot) + (1ull << 48);
  const unsigned long long before = __hip_atomic_fetch_add(words + o, mine, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  if ((int)(before >> 48) == S - 1) {
    R::post(out, o, R::ticket_unpack(before + mine));
    __hip_atomic_store(words + o, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}

template <int NIN, int NOUT, int NEX, int NK, class IT>
struct RowParams {
  char* in[NIN];
  unsigned long long imm[NIN];
  RedOut<NOUT, NEX> out;
  char* partial;          // Acc[S][n_out] when S > 1
  long long n_out;
  long long nblocks;      // blocks of work; more than the grid holds when the plan strides (GS)
  long long nvec;         // vectors in one output's reduce domain (RA * RC / VEC)
  long long chunk;        // vectors per slice
  long long rc_elems;     // elements of one row (UA)
  int S;                  // slices per output
  int pad;
  FastDiv kfd[NK];        // extents of the kept dimensions (slot 0 unused)
  FastDiv rcv;            // RC / VEC, used when RA > 1
  IT kstride[NIN][NK];    // input strides along the kept dimensions
  IT ra_stride[NIN];
  IT rc_stride[NIN];
};

template <class P, int NIN>
struct RedAcc {
  typedef typename P::IT IT;
  char* const* ptr;
  const unsigned long long* imm;
  const IT* vstride;  // stride along the vectorised dimension, per input
  IT off[NIN];

  template <int I, class T, int N>
  THX_DEV void ld(Vec<T, N>& r) const {
    if (P::mode(I) == M_IMM) {
      const T s = *(const T*)&imm[I];
#pragma unroll
      for (int k = 0; k < N; ++k) r.v[k] = s;
      return;
    }
    if (P::mode(I) == M_IOTA) {  // the "strides" of this operand are index multipliers
      const IT st = N > 1 ? vstride[I] : (IT)0;  // the generic form loads single elements and has no vector stride
#pragma unroll
      for (int k = 0; k < N; ++k) r.v[k] = (T)(off[I] + k * st);
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
      const IT st = vstride[I];
#pragma unroll
      for (int k = 0; k < N; ++k) r.v[k] = b[k * st];
    }
  }
};

// Plan members: typedef IT; enum { NK, VEC, UNR, NACC, BLOCK, TPR, RA2 (1 when RA > 1), TICKET, GS, XCD, UA };
// UA: rows whose length is no multiple of VEC, or that do not start on a vector boundary: vectors are read through
// pointers that are only element-aligned, and the RC mod VEC elements at the end of a row one by one.
// static constexpr int mode(int input); static constexpr int sclass(int input, int which).
template <class P, class IT>
THX_DEV IT red_term(int input, int which, IT coord, IT stride) {
  return P::sclass(input, which) == 0 ? (IT)0 : (P::sclass(input, which) == 1 ? coord : coord * stride);
}

// A dispatch carries at most 2^32 - 1 work-items: plans with GS = 1 launch fewer blocks than there is
// work and every block takes the pieces blockIdx.x, blockIdx.x + gridDim.x, ...
template <class R, class P>
__device__ __forceinline__ void red_row_block(const RowParams<R::NIN, R::NOUT, R::NEX, P::NK, typename P::IT>& p, long long bid);

template <class R, class P>
__device__ __forceinline__ void red_row_body(const RowParams<R::NIN, R::NOUT, R::NEX, P::NK, typename P::IT>& p) {
  if constexpr (P::GS != 0) {
    for (long long b = blockIdx.x; b < p.nblocks; b += gridDim.x) {
      red_row_block<R, P>(p, b);
      __syncthreads();
    }
  } else {
    red_row_block<R, P>(p, blockIdx.x);
  }
}

template <class R, class P>
__device__ __forceinline__ void red_row_block(const RowParams<R::NIN, R::NOUT, R::NEX, P::NK, typename P::IT>& p, long long bid) {
  typedef typename P::IT IT;
  typedef typename UnsignedOf<IT>::type UT;
  typedef typename R::Acc Acc;
  constexpr int VEC = P::VEC, UNR = P::UNR, NIN = R::NIN, NK = P::NK, TPR = P::TPR;
  constexpr int RPB = P::BLOCK / TPR;
  __shared__ Acc lds[P::BLOCK / THX_WAVE];

  if constexpr (P::XCD != 0) bid = (bid & 7) * (p.nblocks >> 3) + (bid >> 3);   // a contiguous eighth of the results per die
  const long long ob = bid / p.S;
  const int s = (int)(bid - ob * p.S);
  const long long o = ob * RPB + threadIdx.x / TPR;
  const int t = threadIdx.x % TPR;
  const bool live = o < p.n_out;

  IT base[NIN];
  {
    UT rem = (UT)(live ? o : 0), c;
#pragma unroll
    for (int i = 0; i < NIN; ++i) base[i] = 0;
#pragma unroll
    for (int d = NK - 1; d >= 1; --d) {
      divmod(rem, p.kfd[d], rem, c);
#pragma unroll
      for (int i = 0; i < NIN; ++i) base[i] += (IT)c * p.kstride[i][d];
    }
#pragma unroll
    for (int i = 0; i < NIN; ++i) base[i] += (IT)rem * p.kstride[i][0];
  }

  // UNR vectors are in flight per thread; they are folded into NACC accumulator sets (a set per
  // vector costs registers that long accumulator structs do not leave at 1024 threads per block)
  constexpr int NACC = P::NACC < UNR ? P::NACC : UNR;
  Acc acc[NACC];
#pragma unroll
  for (int u = 0; u < NACC; ++u) R::init(acc[u]);

  if (live) {
    const long long j0 = (long long)s * p.chunk;
    long long j1 = j0 + p.chunk;
    long long nvec = p.nvec;
    if constexpr (P::UA != 0 && P::RA2 == 0) {
      const long long tail0 = nvec * VEC;          // first element of the tail
      if (s == 0) {
        for (long long idx = tail0 + t; idx < p.rc_elems; idx += TPR) {
          typename R::template Regs<1> r1;
          RedAcc<P, NIN> a;
          a.ptr = p.in;
          a.imm = p.imm;
          a.vstride = p.rc_stride;
#pragma unroll
          for (int i = 0; i < NIN; ++i) a.off[i] = base[i] + red_term<P>(i, 1, (IT)idx, p.rc_stride[i]);
          R::template load<1>(a, r1);
          R::template accum<1>(acc[0], r1);
        }
      }
    }
    if (j1 > nvec) j1 = nvec;
    // RA > 1: a thread's vectors are TPR apart, so their (slab, position in the slab) coordinates and every
    // operand's offset advance by the same amounts from one vector to the next - additions and one compare
    // instead of a division and two or three quarter-rate multiplies per vector
    IT cur[NIN], step[NIN], wrap[NIN];
    UT cv = 0, dcv = 0;
    if (P::RA2) {
      UT ra, dra;
      divmod((UT)(j0 + t), p.rcv, ra, cv);
      divmod((UT)TPR, p.rcv, dra, dcv);
#pragma unroll
      for (int i = 0; i < NIN; ++i) {
        const IT along = red_term<P>(i, 1, (IT)VEC, p.rc_stride[i]);      // offset of one vector along RC
        cur[i] = base[i] + red_term<P>(i, 0, (IT)ra, p.ra_stride[i]) + (IT)cv * along;
        step[i] = red_term<P>(i, 0, (IT)dra, p.ra_stride[i]) + (IT)dcv * along;
        wrap[i] = red_term<P>(i, 0, (IT)1, p.ra_stride[i]) - (IT)p.rcv.d * along;
      }
    }
    for (long long j = j0 + t; j < j1; j += (long long)TPR * UNR) {
      typename R::template Regs<VEC> r[UNR];
      bool ok[UNR];
#pragma unroll
      for (int u = 0; u < UNR; ++u) {
        const long long q = j + (long long)u * TPR;
        ok[u] = q < j1;
        RedAcc<P, NIN> a;
        a.ptr = p.in;
        a.imm = p.imm;
        a.vstride = p.rc_stride;
        // P::sclass(input, 0 | 1): the stride along RA | RC is 0, is 1, or anything - a multiply only
        // in the last case (32-bit integer multiplies run at quarter rate)
        if (P::RA2) {
#pragma unroll
          for (int i = 0; i < NIN; ++i) a.off[i] = cur[i];
          if (ok[u]) R::template load<VEC>(a, r[u]);
          // on to the vector TPR further (never dereferenced once it lies beyond the slice)
          cv += dcv;
          const bool over = cv >= p.rcv.d;
          cv -= over ? p.rcv.d : 0;
#pragma unroll
          for (int i = 0; i < NIN; ++i) cur[i] += step[i] + (over ? wrap[i] : (IT)0);
        } else {
#pragma unroll
          for (int i = 0; i < NIN; ++i) a.off[i] = base[i] + red_term<P>(i, 1, (IT)(q * VEC), p.rc_stride[i]);
          if (ok[u]) R::template load<VEC>(a, r[u]);
        }
      }
#pragma unroll
      for (int u = 0; u < UNR; ++u)
        if (ok[u]) R::template accum<VEC>(acc[u % NACC], r[u]);
    }
  }
#pragma unroll
  for (int u = 1; u < NACC; ++u) R::comb(acc[0], acc[u]);

  Acc tot;
  if (TPR > THX_WAVE) {
    tot = block_reduce<R, P::BLOCK / THX_WAVE>(acc[0], lds);
  } else {
    tot = group_reduce<R, TPR>(acc[0]);
  }
  if (p.S == 1) {
    if (live && t == 0) R::post(p.out, o, tot);
    return;
  }
  if constexpr (P::TICKET != 0) {
    if (live && t == 0) ticket_finish<R>(p.out, (unsigned long long*)p.partial, o, p.S, tot);
  } else {
    Acc* part = (Acc*)p.partial;
    if (live && t == 0) part[(long long)s * p.n_out + o] = tot;
  }
}

// ---------------------------------------------------------------------------
// "Column" form: outer kept dims x one or two reduced dims (R rows in all) x
// one kept inner dim (C columns, vectorised). A block is TX x TY threads: TX threads side by
// side along the columns (VEC columns each, so a wave reads whole row segments)
// and TY row lanes; per-column partials live in registers and the TY lanes are
// merged through LDS at the end. Rows are split into S slices.
template <int NIN, int NOUT, int NEX, int NK, class IT>
struct ColParams {
  char* in[NIN];
  unsigned long long imm[NIN];
  RedOut<NOUT, NEX> out;
  char* partial;          // Acc[S][n_out] when S > 1
  long long n_out;        // A * C
  long long nblocks;      // blocks of work; more than the grid holds when the plan strides (GS)
  long long rows;         // R
  long long rows_per_slice;
  int cols;               // C
  int cblocks;            // blocks along the columns
  int S;
  int pad;
  FastDiv kfd[NK];        // extents of the outer kept dimensions (slot 0 unused)
  FastDiv r1;             // extent of the inner reduced dimension, used when RR2
  IT kstride[NIN][NK];
  IT r0_stride[NIN];      // outer reduced dimension (RR2 only)
  IT r1_stride[NIN];      // inner (or only) reduced dimension
  IT c_stride[NIN];
};

// Plan members: typedef IT; enum { NK, VEC, UNR, BLOCK, TX, RR2 (1 when two
// reduced dimensions remain after collapsing), TICKET, GS, UA }; mode(int).
// UA: C is no multiple of VEC, or rows do not start on vector boundaries: element-aligned vector reads, and the
// thread that owns the last, incomplete vector of the columns reads its columns one by one.
template <class R, class P>
__device__ __forceinline__ void red_col_block(const ColParams<R::NIN, R::NOUT, R::NEX, P::NK, typename P::IT>& p, long long bid);

template <class R, class P>
__device__ __forceinline__ void red_col_body(const ColParams<R::NIN, R::NOUT, R::NEX, P::NK, typename P::IT>& p) {
  if constexpr (P::GS != 0) {
    for (long long b = blockIdx.x; b < p.nblocks; b += gridDim.x) {
      red_col_block<R, P>(p, b);
      __syncthreads();
    }
  } else {
    red_col_block<R, P>(p, blockIdx.x);
  }
}

template <class R, class P>
__device__ __forceinline__ void red_col_block(const ColParams<R::NIN, R::NOUT, R::NEX, P::NK, typename P::IT>& p, long long bid) {
  typedef typename P::IT IT;
  typedef typename UnsignedOf<IT>::type UT;
  typedef typename R::Acc Acc;
  constexpr int VEC = P::VEC, UNR = P::UNR, NIN = R::NIN, NK = P::NK, TX = P::TX;
  constexpr int TY = P::BLOCK / TX;
  __shared__ Acc lds[TY][VEC][TX];

  const int cb = (int)(bid % p.cblocks);
  bid /= p.cblocks;
  const int s = (int)(bid % p.S);
  const long long a_idx = bid / p.S;
  const int tx = threadIdx.x % TX, ty = threadIdx.x / TX;
  const int cv = cb * TX + tx;                 // column vector owned by this thread
  const bool live = (long long)cv * VEC < p.cols;
  // UA: the last vector of a row that is no whole number of vectors ends with the row and overlaps its
  // neighbour; the columns it repeats are dropped when the results are written
  const int c0 = P::UA != 0 && live && cv * VEC + VEC > p.cols && p.cols >= VEC ? p.cols - VEC : cv * VEC;

  IT base[NIN];
  {
    UT rem = (UT)a_idx, c;
#pragma unroll
    for (int i = 0; i < NIN; ++i) base[i] = (IT)(live ? c0 : 0) * p.c_stride[i];
#pragma unroll
    for (int d = NK - 1; d >= 1; --d) {
      divmod(rem, p.kfd[d], rem, c);
#pragma unroll
      for (int i = 0; i < NIN; ++i) base[i] += (IT)c * p.kstride[i][d];
    }
#pragma unroll
    for (int i = 0; i < NIN; ++i) base[i] += (IT)rem * p.kstride[i][0];
  }

  Acc acc[VEC];
#pragma unroll
  for (int k = 0; k < VEC; ++k) R::init(acc[k]);

  if (live) {
    const long long r0 = (long long)s * p.rows_per_slice;
    long long r1 = r0 + p.rows_per_slice;
    if (r1 > p.rows) r1 = p.rows;
    for (long long rr = r0 + ty; rr < r1; rr += (long long)TY * UNR) {
      typename R::template Regs<VEC> r[UNR];
      bool ok[UNR];
#pragma unroll
      for (int u = 0; u < UNR; ++u) {
        const long long q = rr + (long long)u * TY;
        ok[u] = q < r1;
        RedAcc<P, NIN> a;
        a.ptr = p.in;
        a.imm = p.imm;
        a.vstride = p.c_stride;
        if (P::RR2) {
          UT q0, q1;
          divmod((UT)(ok[u] ? q : r0), p.r1, q0, q1);
#pragma unroll
          for (int i = 0; i < NIN; ++i)
            a.off[i] = base[i] + (IT)q0 * p.r0_stride[i] + (IT)q1 * p.r1_stride[i];
        } else {
#pragma unroll
          for (int i = 0; i < NIN; ++i) a.off[i] = base[i] + (IT)q * p.r1_stride[i];
        }
        if (ok[u]) R::template load<VEC>(a, r[u]);
      }
#pragma unroll
      for (int u = 0; u < UNR; ++u)
        if (ok[u]) R::template accum_lanes<VEC>(acc, r[u]);
    }
  }

#pragma unroll
  for (int k = 0; k < VEC; ++k) lds[ty][k][tx] = acc[k];
  __syncthreads();
  Acc* part = (Acc*)p.partial;
  for (int c = threadIdx.x; c < TX * VEC; c += P::BLOCK) {
    const int x = c / VEC;
    int k = c % VEC;
    const long long col = (long long)cb * (TX * VEC) + c;
    if (col < p.cols) {
      if constexpr (P::UA != 0) {
        const long long first = col - k;                   // first column of this vector, had it not been moved
        if (first + VEC > p.cols) k = (int)(col - (p.cols - VEC));
      }
      Acc tot = lds[0][k][x];
#pragma unroll
      for (int y = 1; y < TY; ++y) R::comb(tot, lds[y][k][x]);
      const long long o = a_idx * p.cols + col;
      if (p.S == 1) {
        R::post(p.out, o, tot);
      } else if constexpr (P::TICKET != 0) {
        ticket_finish<R>(p.out, (unsigned long long*)p.partial, o, p.S, tot);
      } else {
        part[(long long)s * p.n_out + o] = tot;
      }
    }
  }
}

// ---------------------------------------------------------------------------
// "Strip" form: a C-contiguous (rows, C) array with fewer columns than a few vectors hold, reduced over the rows
// (per-coordinate sums of n points in 3 dimensions).  The array is walked as the flat run of rows * C elements it
// is, in whole vectors, consecutive threads on consecutive vectors.  A block takes C * BLOCK vectors at a time: a
// thread's vector in step u is u * BLOCK vectors after its first, so its element j lies in column
// (first + u * (BLOCK * VEC mod C) + j) mod C, where `first` - the column of the thread's very first element -
// is the same in every round of C steps.  With the steps unrolled every accumulator index is a constant (relative
// to `first`); the rotation by `first` happens once, when the accumulators go to LDS.
template <int NIN, int NOUT, int NEX>
struct StripParams {
  char* in[NIN];
  unsigned long long imm[NIN];
  RedOut<NOUT, NEX> out;
  char* partial;          // Acc[blocks][C] when there is more than one block
  long long nvec;         // whole vectors in the array
  long long n;            // elements in the array (rows * C)
  int blocks;
  int pad;
};

// Plan members: typedef IT; enum { VEC, COLS, BLOCK, UA }; mode(int) (M_VEC or M_IMM only).
template <class R, class P>
__device__ __forceinline__ void red_strip_body(const StripParams<R::NIN, R::NOUT, R::NEX>& p) {
  typedef typename P::IT IT;
  typedef typename R::Acc Acc;
  constexpr int VEC = P::VEC, C = P::COLS, NIN = R::NIN, BLOCK = P::BLOCK;
  constexpr int DELTA = (BLOCK * VEC) % C;
  __shared__ Acc lds[C][BLOCK];

  const int t = threadIdx.x;
  const int first = (int)(((long long)t * VEC) % C);
  Acc acc[C];
#pragma unroll
  for (int i = 0; i < C; ++i) R::init(acc[i]);

  const IT no_stride[NIN] = {};
  for (long long q0 = (long long)blockIdx.x * (C * BLOCK); q0 < p.nvec; q0 += (long long)gridDim.x * (C * BLOCK)) {
    typename R::template Regs<VEC> r[C];
    bool ok[C];
#pragma unroll
    for (int u = 0; u < C; ++u) {
      const long long q = q0 + (long long)u * BLOCK + t;
      ok[u] = q < p.nvec;
      RedAcc<P, NIN> a;
      a.ptr = p.in;
      a.imm = p.imm;
      a.vstride = no_stride;
#pragma unroll
      for (int i = 0; i < NIN; ++i) a.off[i] = (IT)(q * VEC);
      if (ok[u]) R::template load<VEC>(a, r[u]);
    }
#pragma unroll
    for (int u = 0; u < C; ++u) {
      if (ok[u]) {
        Acc lane[VEC];
#pragma unroll
        for (int j = 0; j < VEC; ++j) R::init(lane[j]);
        R::template accum_lanes<VEC>(lane, r[u]);
#pragma unroll
        for (int j = 0; j < VEC; ++j) R::comb(acc[(u * DELTA + j) % C], lane[j]);
      }
    }
  }

#pragma unroll
  for (int i = 0; i < C; ++i) {
    int c = first + i;
    if (c >= C) c -= C;
    lds[c][t] = acc[i];
  }
  __syncthreads();
  const int wave = t / THX_WAVE, lane_id = t % THX_WAVE;
  for (int c = wave; c < C; c += BLOCK / THX_WAVE) {
    Acc tot = lds[c][lane_id];
#pragma unroll
    for (int k = 1; k < BLOCK / THX_WAVE; ++k) R::comb(tot, lds[c][lane_id + k * THX_WAVE]);
    tot = group_reduce<R, THX_WAVE>(tot);
    if (lane_id == 0) {
      if (blockIdx.x == 0) {       // the elements after the last whole vector
        for (long long e = p.nvec * VEC; e < p.n; ++e) {
          if ((int)(e % C) != c) continue;
          typename R::template Regs<1> r1;
          RedAcc<P, NIN> a;
          a.ptr = p.in;
          a.imm = p.imm;
          a.vstride = no_stride;
#pragma unroll
          for (int i = 0; i < NIN; ++i) a.off[i] = (IT)e;
          R::template load<1>(a, r1);
          R::template accum<1>(tot, r1);
        }
      }
      if (p.blocks == 1) R::post(p.out, c, tot);
      else ((Acc*)p.partial)[(long long)blockIdx.x * C + c] = tot;
    }
  }
}

// ---------------------------------------------------------------------------
// Second pass: merge the S partial Acc values of every output, slice 0 first.
// TPO threads per output (1, 64 or BLOCK).
template <int NOUT, int NEX>
struct FinalParams {
  RedOut<NOUT, NEX> out;
  char* partial;
  long long n_out;
  int S;
  int pad;
};

template <class R, int BLOCK, int TPO>
__device__ __forceinline__ void red_final_body(const FinalParams<R::NOUT, R::NEX>& p) {
  typedef typename R::Acc Acc;
  __shared__ Acc lds[BLOCK / THX_WAVE];
  const Acc* part = (const Acc*)p.partial;
  const long long o = (long long)blockIdx.x * (BLOCK / TPO) + threadIdx.x / TPO;
  const int t = threadIdx.x % TPO;
  const bool live = o < p.n_out;
  Acc acc;
  R::init(acc);
  if (live)
    for (int s = t; s < p.S; s += TPO) R::comb(acc, part[(long long)s * p.n_out + o]);
  if (TPO > THX_WAVE) {
    acc = block_reduce<R, BLOCK / THX_WAVE>(acc, lds);
  } else if (TPO > 1) {
    acc = group_reduce<R, TPO>(acc);
  }
  if (live && t == 0) R::post(p.out, o, acc);
}

// ---------------------------------------------------------------------------
// Fallback for any mask that does not collapse to the row or column form: TPR
// threads per output walk the flattened reduce domain and decompose every
// index. Correct for every pattern, coalesced only by luck.
template <int NIN, int NOUT, int NEX, int NK, int NR, class IT>
struct GenParams {
  char* in[NIN];
  unsigned long long imm[NIN];
  RedOut<NOUT, NEX> out;
  long long n_out;
  long long nblocks;      // blocks of work; more than the grid holds when the plan strides (GS)
  long long n_red;
  FastDiv kfd[NK];
  FastDiv rfd[NR];
  IT kstride[NIN][NK];
  IT rstride[NIN][NR];
};

// Plan members: typedef IT; enum { NK, NR, BLOCK, TPR, GS }.
template <class R, class P>
__device__ __forceinline__ void red_gen_block(const GenParams<R::NIN, R::NOUT, R::NEX, P::NK, P::NR, typename P::IT>& p, long long bid);

template <class R, class P>
__device__ __forceinline__ void red_gen_body(const GenParams<R::NIN, R::NOUT, R::NEX, P::NK, P::NR, typename P::IT>& p) {
  if constexpr (P::GS != 0) {
    for (long long b = blockIdx.x; b < p.nblocks; b += gridDim.x) {
      red_gen_block<R, P>(p, b);
      __syncthreads();
    }
  } else {
    red_gen_block<R, P>(p, blockIdx.x);
  }
}

template <class R, class P>
__device__ __forceinline__ void red_gen_block(const GenParams<R::NIN, R::NOUT, R::NEX, P::NK, P::NR, typename P::IT>& p, long long bid) {
  typedef typename P::IT IT;
  typedef typename UnsignedOf<IT>::type UT;
  typedef typename R::Acc Acc;
  constexpr int NIN = R::NIN, NK = P::NK, NR = P::NR, TPR = P::TPR;
  __shared__ Acc lds[P::BLOCK / THX_WAVE];
  const long long o = bid * (P::BLOCK / TPR) + threadIdx.x / TPR;
  const int t = threadIdx.x % TPR;
  const bool live = o < p.n_out;
  IT base[NIN];
  {
    UT rem = (UT)(live ? o : 0), c;
#pragma unroll
    for (int i = 0; i < NIN; ++i) base[i] = 0;
#pragma unroll
    for (int d = NK - 1; d >= 1; --d) {
      divmod(rem, p.kfd[d], rem, c);
#pragma unroll
      for (int i = 0; i < NIN; ++i) base[i] += (IT)c * p.kstride[i][d];
    }
#pragma unroll
    for (int i = 0; i < NIN; ++i) base[i] += (IT)rem * p.kstride[i][0];
  }
  Acc acc;
  R::init(acc);
  if (live) {
    for (long long j = t; j < p.n_red; j += TPR) {
      UT rem = (UT)j, c;
      RedAcc<P, NIN> a;
      a.ptr = p.in;
      a.imm = p.imm;
      a.vstride = nullptr;
#pragma unroll
      for (int i = 0; i < NIN; ++i) a.off[i] = base[i];
#pragma unroll
      for (int d = NR - 1; d >= 1; --d) {
        divmod(rem, p.rfd[d], rem, c);
#pragma unroll
        for (int i = 0; i < NIN; ++i) a.off[i] += (IT)c * p.rstride[i][d];
      }
#pragma unroll
      for (int i = 0; i < NIN; ++i) a.off[i] += (IT)rem * p.rstride[i][0];
      typename R::template Regs<1> r;
      R::template load<1>(a, r);
      R::template accum<1>(acc, r);
    }
  }
  if (TPR > THX_WAVE) {
    acc = block_reduce<R, P::BLOCK / THX_WAVE>(acc, lds);
  } else if (TPR > 1) {
    acc = group_reduce<R, TPR>(acc);
  }
  if (live && t == 0) R::post(p.out, o, acc);
}

}  // namespace thx
