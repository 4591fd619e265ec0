// Elementwise planner: validates operands, collapses dimensions, picks an
// access plan (rank, index width, vector width, per-operand access mode),
// compiles the matching kernel on first use and launches it.
#include <algorithm>
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <sstream>
#include <unordered_map>

#include "thx_internal.h"

namespace thx {

enum { M_VEC = 0, M_BCAST = 1, M_GATHER = 2, M_IMM = 3 };

static int64_t ceil_div64(int64_t a, int64_t b) { return (a + b - 1) / b; }

struct Dims {
  int nd = 0;
  int64_t shape[THX_MAX_ND];
  std::vector<std::vector<int64_t>> stride;  // [operand][dim]
};

// Drop extent-1 dimensions, then merge neighbours (outer d, inner d+1) that
// every operand walks as one: stride[d] == stride[d+1] * shape[d+1].
static void collapse(Dims* d) {
  const size_t nops = d->stride.size();
  int w = 0;
  for (int i = 0; i < d->nd; ++i) {
    if (d->shape[i] == 1) continue;
    d->shape[w] = d->shape[i];
    for (size_t o = 0; o < nops; ++o) d->stride[o][w] = d->stride[o][i];
    ++w;
  }
  d->nd = w;
  if (w == 0) {
    d->nd = 1;
    d->shape[0] = 1;
    for (size_t o = 0; o < nops; ++o) d->stride[o][0] = 0;
    return;
  }
  int out = 0;  // index of the dimension being grown
  for (int i = 1; i < d->nd; ++i) {
    bool ok = true;
    for (size_t o = 0; o < nops && ok; ++o) ok = d->stride[o][out] == d->stride[o][i] * d->shape[i];
    if (ok) {
      d->shape[out] *= d->shape[i];
      for (size_t o = 0; o < nops; ++o) d->stride[o][out] = d->stride[o][i];
    } else {
      ++out;
      d->shape[out] = d->shape[i];
      for (size_t o = 0; o < nops; ++o) d->stride[o][out] = d->stride[o][i];
    }
  }
  d->nd = out + 1;
}

static int env_int(const char* name, int dflt) {
  const char* v = getenv(name);
  return v ? atoi(v) : dflt;
}

}  // namespace thx

using namespace thx;

extern "C" {

int thx_elemwise_new(const char* functor_src, const char* functor_name, int n_in, int n_out, const int32_t* dtypes,
                     thx_elemwise** out) {
  if (!functor_src || !functor_name || !dtypes || !out) return fail(THX_ERR_ARG, "thx_elemwise_new: null argument");
  if (n_in < 1 || n_out < 1) return fail(THX_ERR_ARG, "thx_elemwise_new: needs inputs and outputs");
  for (int i = 0; i < n_in + n_out; ++i)
    if (!dtype_size(dtypes[i])) return fail(THX_ERR_TYPE, "thx_elemwise_new: unknown dtype code %d", dtypes[i]);
  thx_elemwise* e = new thx_elemwise;
  e->src = functor_src;
  e->name = functor_name;
  e->n_in = n_in;
  e->n_out = n_out;
  e->dtypes.assign(dtypes, dtypes + n_in + n_out);
  *out = e;
  return THX_OK;
}

int thx_elemwise_free(thx_elemwise* e) {
  delete e;
  return THX_OK;
}

}  // extern "C"

// thx_elemwise_call and thx_elemwise_reduce_call.  With `red_outs` the operation's attached reduction is
// computed as well: inside the permuted-read kernel when that plan is taken and the results' innermost
// dimension is the one the reduction keeps (*fused = true), otherwise the caller reduces the stored results.
static int elemwise_impl(thx_elemwise* e, const thx_array* ins, const thx_array* outs, const thx_array* red_outs,
                         int flags, bool* fused) {
  if (!e || !ins || !outs) return fail(THX_ERR_ARG, "thx_elemwise_call: null argument");
  const bool dry = (flags & THX_DRY_RUN) != 0;
  if (!dry) {
    int rc = ensure_init();
    if (rc) return rc;
  }
  const int nops = e->n_in + e->n_out;
  int nd = 0;
  int64_t shape[THX_MAX_ND];
  std::vector<View> views;
  int rc = gather_inputs("elemwise", ins, e->n_in, e->dtypes.data(), flags, &nd, shape, &views);
  if (rc) return rc;
  // Inputs that all have extent 1 along a dimension broadcast to the outputs' extent there
  // (a fill: every input is a scalar and the output alone carries the shape).
  if ((flags & THX_BROADCAST) && e->n_out > 0 && outs[0].nd == nd) {
    for (int d = 0; d < nd; ++d) {
      if (shape[d] == 1 && outs[0].shape[d] != 1) {
        shape[d] = outs[0].shape[d];
        for (int i = 0; i < e->n_in; ++i) views[i].stride[d] = 0;
      }
    }
  }
  views.resize(nops);
  for (int o = 0; o < e->n_out; ++o) {
    const thx_array& a = outs[o];
    View& v = views[e->n_in + o];
    if (a.nd != nd) return fail(THX_ERR_TYPE, "elemwise: output %d has rank %d, expected %d", o, a.nd, nd);
    const int adt = a.dtype & ~THX_REUSED;
    if (adt != e->dtypes[e->n_in + o])
      return fail(THX_ERR_TYPE, "elemwise: output %d has dtype code %d, the operation was built for %d", o, adt,
                  e->dtypes[e->n_in + o]);
    const int isz = dtype_size(adt);
    if (null_base(a, dry)) return fail(THX_ERR_ARG, "elemwise: output %d has no base address", o);
    v.ptr = (char*)a.base + a.offset_bytes;
    v.dtype = adt;
    v.reused = (a.dtype & THX_REUSED) != 0;
    if (((uintptr_t)v.ptr) % isz) return fail(THX_ERR_TYPE, "elemwise: output %d is not aligned to its element size", o);
    for (int d = 0; d < nd; ++d) {
      if (a.shape[d] != shape[d])
        return fail(THX_ERR_SHAPE, "elemwise: output %d has extent %lld along dimension %d, the result has %lld", o,
                    (long long)a.shape[d], d, (long long)shape[d]);
      if (a.strides_bytes[d] % isz)
        return fail(THX_ERR_TYPE, "elemwise: output %d stride is not a multiple of its element size", o);
      v.stride[d] = a.strides_bytes[d] / isz;
      if (shape[d] > 1 && v.stride[d] == 0)
        return fail(THX_ERR_TYPE, "elemwise: output %d has a zero stride along dimension %d", o, d);
    }
  }
  for (int o = 0; o < e->n_in; ++o)
    if (views[o].iota) return fail(THX_ERR_UNSUPPORTED, "elemwise: index operands are for reductions only");
  int64_t n = 1;
  for (int d = 0; d < nd; ++d) n *= shape[d];
  if (n == 0) {
    set_last_plan("ew|empty");
    return THX_OK;
  }

  Dims dm;
  dm.nd = nd;
  for (int d = 0; d < nd; ++d) dm.shape[d] = shape[d];
  dm.stride.resize(nops);
  for (int o = 0; o < nops; ++o) dm.stride[o].assign(views[o].stride, views[o].stride + THX_MAX_ND);
  if (nd == 0) {
    dm.nd = 1;
    dm.shape[0] = 1;
    for (int o = 0; o < nops; ++o) dm.stride[o][0] = 0;
  }
  // Dimensions in the order of the first result's strides, largest first: operands that share a permuted layout
  // (every one of them a transposed view, the result allocated to match) then collapse and vectorise like
  // C-contiguous ones instead of walking memory with the longest stride innermost.  A C-ordered result keeps its
  // order; the variant that reduces while it stores relies on that order and is left alone.
  if (dm.nd > 1 && !(red_outs && e->red)) {
    const std::vector<int64_t>& os = dm.stride[e->n_in];
    std::vector<int> order(dm.nd);
    for (int d = 0; d < dm.nd; ++d) order[d] = d;
    // (extent-1 dimensions, whose strides mean nothing, go first: the collapse drops them)
    auto mag = [&](int d) { return dm.shape[d] == 1 ? INT64_MAX : (os[d] < 0 ? -os[d] : os[d]); };
    std::stable_sort(order.begin(), order.end(), [&](int a, int b) { return mag(a) > mag(b); });
    bool moved = false;
    for (int d = 0; d < dm.nd; ++d) moved = moved || order[d] != d;
    if (moved) {
      int64_t shp[THX_MAX_ND];
      for (int d = 0; d < dm.nd; ++d) shp[d] = dm.shape[order[d]];
      for (int d = 0; d < dm.nd; ++d) dm.shape[d] = shp[d];
      for (int o = 0; o < nops; ++o) {
        std::vector<int64_t> st(dm.stride[o]);
        for (int d = 0; d < dm.nd; ++d) dm.stride[o][d] = st[order[d]];
      }
    }
  }
  collapse(&dm);
  const int ND = dm.nd;
  const int64_t inner = dm.shape[ND - 1];

  // index width: every element offset and the flat index must fit in 31 bits
  bool wide = n >= (int64_t(1) << 31) - 65536;
  for (int o = 0; o < nops && !wide; ++o) {
    int64_t span = 0;
    for (int d = 0; d < ND; ++d) span += (dm.shape[d] - 1) * (dm.stride[o][d] < 0 ? -dm.stride[o][d] : dm.stride[o][d]);
    if (span >= (int64_t(1) << 31) - 65536) wide = true;
  }

  // access modes along the innermost dimension
  std::vector<int> mode(nops);
  int maxsz = 0;
  bool any_vec = false;
  for (int o = 0; o < nops; ++o) {
    const int64_t st = dm.stride[o][ND - 1];
    mode[o] = st == 1 ? M_VEC : (st == 0 ? M_BCAST : M_GATHER);
    if (n == 1) mode[o] = M_BCAST;
    if (views[o].imm) mode[o] = M_IMM;
    if (o >= e->n_in && mode[o] == M_BCAST) mode[o] = M_GATHER;
    if (mode[o] == M_VEC) {
      any_vec = true;
      if (dtype_size(views[o].dtype) > maxsz) maxsz = dtype_size(views[o].dtype);
    }
  }
  int vec = any_vec ? 16 / maxsz : 1;
  const int force_vec = env_int("THX_EW_VEC", 0);
  if (force_vec > 0 && force_vec < vec) vec = force_vec;
  auto vec_ok = [&](int v) {
    if (v == 1) return true;
    if (ND > 1 && (inner % v != 0 || inner / v < 2)) return false;
    for (int o = 0; o < nops; ++o) {
      if (mode[o] != M_VEC) continue;
      const int isz = dtype_size(views[o].dtype);
      if (((uintptr_t)views[o].ptr) % (size_t)(isz * v)) return false;
      for (int d = 0; d < ND - 1; ++d)
        if (dm.stride[o][d] % v) return false;
    }
    return true;
  };
  const int vec_full = vec;
  while (!vec_ok(vec)) vec /= 2;
  // Operands that start off a vector boundary, or whose rows do (views that drop a first element or column; float16
  // and int8 suffer most from narrow accesses): full-width vectors through element-aligned pointers.
  int ua = 0;
  if (vec < vec_full && env_int("THX_EW_UA", 1)) {
    auto ua_ok = [&](int v) {
      if (ND > 1 && (inner % v != 0 || inner / v < 2)) return false;
      for (int o = 0; o < nops; ++o)
        if (mode[o] == M_VEC && ((uintptr_t)views[o].ptr) % (size_t)dtype_size(views[o].dtype)) return false;
      return true;
    };
    int v = vec_full;
    while (v > vec && !ua_ok(v)) v /= 2;
    if (v > vec) {
      vec = v;
      ua = 1;
    }
  }
  // Rows that are no whole number of vectors ((n, 1001) plus a row that broadcasts): the thread that owns the last,
  // incomplete vector of a row handles its elements one by one; rows of 16 vectors and more.
  int rag = 0;
  if (vec < vec_full && ND > 1 && env_int("THX_EW_UA", 1) && env_int("THX_EW_RAGGED", 1)) {
    bool ok = true;
    for (int o = 0; o < nops; ++o)
      if (mode[o] == M_VEC && ((uintptr_t)views[o].ptr) % (size_t)dtype_size(views[o].dtype)) ok = false;
    int v = vec_full;
    while (v > vec && inner < (int64_t)v * 16) v /= 2;
    if (ok && v > vec && inner % v != 0) {
      vec = v;
      ua = 1;
      rag = 1;
    }
  }
  const int64_t row_vecs = ND > 1 ? (inner + vec - 1) / vec : 0;   // vectors in a row, the incomplete one included

  // bytes the kernel moves: every operand that is not broadcast along the innermost dimension
  int64_t moved = 0;
  for (int o = 0; o < nops; ++o)
    if (mode[o] == M_VEC || mode[o] == M_GATHER) moved += n * dtype_size(views[o].dtype);

  // permuted-read plan: inputs that are unit-stride along another dimension T go through LDS tiles
  if (ND >= 2 && !wide && !env_int("THX_EW_NO_TRANSPOSE", 0)) {
    bool any_gather = false, outs_ok = true;
    for (int o = 0; o < nops; ++o) {
      if (o < e->n_in && mode[o] == M_GATHER) any_gather = true;
      if (o >= e->n_in && mode[o] != M_VEC) outs_ok = false;
    }
    int tdim = -1;
    if (any_gather && outs_ok && inner >= 16) {
      for (int d = ND - 2; d >= 0 && tdim < 0; --d) {
        if (dm.shape[d] < 16) continue;
        bool ok = true;
        for (int o = 0; o < e->n_in && ok; ++o)
          if (mode[o] == M_GATHER && dm.stride[o][d] != 1) ok = false;
        if (ok) tdim = d;
      }
    }
    if (tdim >= 0) {
      std::vector<int> slot(nops, -1);
      int ntr = 0, esz = 1;
      for (int o = 0; o < e->n_in; ++o)
        if (mode[o] == M_GATHER) {
          slot[o] = ntr++;
          esz = std::max(esz, dtype_size(views[o].dtype));
        }
      // 128-byte row segments are enough for the memory system, and the smaller tile keeps four times
      // as many blocks in flight around the barrier between the two phases: 53.0 us against 60.0 us for
      // the int32 (64, 128, 56, 56) permuted read with 64 x 64 tiles
      int tile = esz >= 4 ? 32 : 64;
      if ((int64_t)ntr * tile * (tile + 1) * esz > 60000) tile = 32;
      const int force_tile = env_int("THX_EW_TILE", 0);
      if (force_tile == 32 || force_tile == 64) tile = force_tile;
      // extents of the tile along T (rows read from the permuted inputs) and along the inner dimension
      int tile_t = tile, tile_i = tile;
      // More operands walk the inner dimension (the results and the inputs that are not permuted) than are
      // permuted: 512-byte segments for them and 128-byte rows for the permuted reads - x.T * 2 + y on
      // (8192, 8192) float32 5.6 TB/s against 4.4 with the square tile, (8191, 8193) 4.4 against 2.8 (rows that do
      // not start on cache lines waste less of a longer segment), float16 4.9 / 3.2 against 4.8 / 2.4.  With the
      // permuted reads in the majority (two of them and one result: the (64, 128, 56, 56) case) the square tile
      // ties with every other shape measured.
      {
        int along_inner = 0;
        for (int o = 0; o < nops; ++o)
          if (!views[o].imm && slot[o] < 0 && mode[o] != M_BCAST) ++along_inner;
        if (along_inner > ntr && (inner + 127) / 128 * 128 * 100 <= inner * 115 && !red_outs && env_int("THX_EW_WIDE_TILE", 1) &&
            (int64_t)ntr * 128 * (32 + 1) * esz <= 60000) {
          tile_t = 32;
          tile_i = 128;
        }
      }
      {
        const int ft = env_int("THX_EW_TILE_T", 0), fi = env_int("THX_EW_TILE_I", 0);
        auto pow2 = [](int v) { return v >= 8 && v <= 256 && (v & (v - 1)) == 0; };
        if (pow2(ft) && pow2(fi) && ft * fi >= 1024) {
          tile_t = ft;
          tile_i = fi;
        }
      }
      // elements per access: 16 bytes of the widest operand, if extents, strides and addresses allow
      int allsz = 1;
      for (int o = 0; o < nops; ++o)
        if (!views[o].imm) allsz = std::max(allsz, dtype_size(views[o].dtype));
      int tv = std::min(4, 16 / allsz);
      auto tv_ok = [&](int v) {
        if (v == 1) return true;
        if (dm.shape[tdim] % v || inner % v) return false;
        for (int o = 0; o < nops; ++o) {
          if (views[o].imm) continue;
          const bool staged = slot[o] >= 0;
          if (!staged && mode[o] != M_VEC) continue;  // broadcast operands are read one element at a time
          if (((uintptr_t)views[o].ptr) % (size_t)(dtype_size(views[o].dtype) * v)) return false;
          for (int d = 0; d < ND; ++d) {
            if (staged ? d == tdim : d == ND - 1) continue;
            if (dm.stride[o][d] % v) return false;
          }
        }
        return true;
      };
      while (!tv_ok(tv)) tv /= 2;
      if (env_int("THX_EW_TV", 0) == 1) tv = 1;
      // Extents or strides that leave single-element accesses, 4-byte elements and wider: the rows of a tile do
      // not start on cache lines, and a longer segment along the inner dimension wastes less of them - also when the
      // permuted reads are not in the minority ((255, 513, 511) float32, one permuted read and one result:
      // 1.7 - 2.2 TB/s with the square tile, 2.9 with 32 x 128; 2-byte elements lose with it)
      if (tv == 1 && esz >= 4 && tile_t == tile && tile_i == tile && (inner + 127) / 128 * 128 * 100 <= inner * 115 && !red_outs && env_int("THX_EW_WIDE_TILE", 1) &&
          !env_int("THX_EW_TILE_T", 0) && (int64_t)ntr * 128 * (32 + 1) * esz <= 60000) {
        int along_inner = 0;
        for (int o = 0; o < nops; ++o)
          if (!views[o].imm && slot[o] < 0 && mode[o] != M_BCAST) ++along_inner;
        if (along_inner >= ntr) {
          tile_t = 32;
          tile_i = 128;
        }
      }
      if ((int64_t)ntr * tile_i * (tile_t + 1) * esz <= 60000) {
        const int block = 256;
        // the attached reduction rides along when it keeps exactly the innermost dimension of the results
        // (which the collapse must have left alone) and the row lanes of a block fit the LDS
        thx_reduce* R = red_outs ? e->red : nullptr;
        const int rpp_c = block / (tile_i / tv);
        const bool red = R && !env_int("THX_EW_NO_FUSED_REDUCE", 0) && nd >= 2 && inner == shape[nd - 1] &&
                         tile_t % rpp_c == 0 && (int64_t)rpp_c * tile_i * R->acc_bytes <= 60000;
        if (R && !red)   // the caller reduces the stored results next: they stay cacheable
          for (int w : e->red_of) views[e->n_in + w].reused = true;
        const uint64_t nt = nt_mask(nt_streaming(moved), views);
        // Measured on the int32 (64, 128, 56, 56) permuted read and left off: two tile buffers (one barrier per
        // tile instead of two) change nothing, 58.9 us against 58.8 us with the channel sum attached; resident
        // blocks that stride over the tiles with the next tile's loads in flight match one block per tile at 4-6
        // blocks per compute unit (53.2-53.5 us against 53.5 us) and lose at 8 (56.1 us).
        const int64_t lds_one = (int64_t)ntr * tile_i * (tile_t + 1) * esz;
        const int nbuf = (2 * lds_one <= 60000 && env_int("THX_EW_TR_NBUF", 1) == 2) ? 2 : 1;
        const bool persist = !red && env_int("THX_EW_TR_PERSIST", 0) != 0;
        std::ostringstream key;
        key << (red ? "er|nd" : "et|nd") << ND << "|t" << tile_t << "x" << tile_i << "|v" << tv << "|n" << ntr << "|e" << esz
            << (nbuf == 2 ? "|b2" : "") << (persist ? "|p" : "");
        if (nt) key << "|nt" << std::hex << nt << std::dec;
        key << "|m";
        for (int o = 0; o < nops; ++o) key << (slot[o] >= 0 ? 9 : mode[o]) << (o + 1 < nops ? "," : "");
        const std::string plan = key.str() + (fast_div() ? "|fd" : "");
        set_last_plan(e->name + "|" + plan);
        Kernel k;
        auto it = e->plans.find(plan);
        if (it != e->plans.end() && (it->second.func || dry)) {
          k = it->second;
        } else {
          const std::string entry = entry_name(e->name, plan);
          std::ostringstream s;
          s << device_prelude() << e->src << "\nstruct ThxPlan {\n  typedef int IT;\n  enum { ND = " << ND
            << ", TT = " << tile_t << ", TI = " << tile_i << ", TV = " << tv << ", BLOCK = " << block << ", NTR = " << ntr << ", ESZ = " << esz
            << ", RED = " << (red ? 1 : 0) << ", NBUF = " << nbuf << ", PERSIST = " << (persist ? 1 : 0)
            << " };\n  static constexpr unsigned long long NT = " << nt << "ull;\n  static constexpr int mode(int i) {\n    constexpr int m[] = {";
          for (int o = 0; o < nops; ++o) s << mode[o] << (o + 1 < nops ? ", " : "");
          s << "};\n    return m[i];\n  }\n  static constexpr int slot(int i) {\n    constexpr int m[] = {";
          for (int o = 0; o < nops; ++o) s << slot[o] << (o + 1 < nops ? ", " : "");
          s << "};\n    return m[i];\n  }\n};\n";
          if (red)
            s << "extern \"C\" __global__ __launch_bounds__(" << block << ") void " << entry << "(thx::EwTrParams<" << e->name
              << "::NOPS, ThxPlan::ND, ThxPlan::IT> p, thx::EwRedParams<" << R->name << "::NOUT, " << R->name
              << "::NEX> q) {\n  thx::ew_tr_red_body<" << e->name << ", ThxPlan>(p, q);\n}\n";
          else
            s << "extern \"C\" __global__ __launch_bounds__(" << block << ") void " << entry << "(thx::EwTrParams<" << e->name
              << "::NOPS, ThxPlan::ND, ThxPlan::IT> p, unsigned total) {\n  thx::ew_tr_body<" << e->name << ", ThxPlan>(p, total);\n}\n";
          rc = get_kernel(s.str(), entry, &k);
          if (rc) return rc;
          e->plans[plan] = k;
        }
        const int64_t ext_t = dm.shape[tdim], ext_i = inner;
        const int64_t tiles_t = (ext_t + tile_t - 1) / tile_t, tiles_i = (ext_i + tile_i - 1) / tile_i;
        int64_t outer = 1;
        std::vector<int> odims;
        for (int d = 0; d < ND - 1; ++d)
          if (d != tdim) {
            odims.push_back(d);
            outer *= dm.shape[d];
          }
        // reducing variant: `groups` blocks share one innermost range and split the other tiles evenly
        const int64_t rowtiles = outer * tiles_t;
        int64_t groups = 1;
        if (red) {
          const int64_t cus = rt().ready ? rt().cus : 256;
          const int bpc = std::max(1, env_int("THX_EW_RED_BLOCKS_PER_CU", 4));  // 3 to 6 measured within 1 %, 8 and 2 worse (partials stay few)
          const int64_t g0 = std::max<int64_t>(1, std::min(rowtiles, cus * bpc / tiles_i));
          groups = ceil_div64(rowtiles, ceil_div64(rowtiles, g0));
        }
        std::vector<char*> routp;
        std::vector<uint64_t> rex(1, 0);
        std::vector<int64_t> rexs(1, 1);
        if (red) {
          for (int o = 0; o < R->n_out; ++o) {
            const thx_array& a = red_outs[o];
            const int adt = a.dtype & ~THX_REUSED;
            int64_t count = 1;
            for (int d = 0; d < a.nd; ++d) count *= a.shape[d];
            int64_t expect = dtype_size(adt);
            bool contiguous = true;
            for (int d = a.nd - 1; d >= 0; --d) {
              if (a.shape[d] > 1 && a.strides_bytes[d] != expect) contiguous = false;
              expect *= a.shape[d];
            }
            if (adt != R->dtypes[R->n_in + o] || count != ext_i || !contiguous)
              return fail(THX_ERR_TYPE, "elemwise: reduction result %d must be a C-contiguous array of %lld elements of "
                          "dtype code %d", o, (long long)ext_i, R->dtypes[R->n_in + o]);
            if (null_base(a, dry)) return fail(THX_ERR_ARG, "elemwise: reduction result %d has no base address", o);
            routp.push_back((char*)a.base + a.offset_bytes);
          }
          if (rowtiles >= (int64_t(1) << 31)) return fail(THX_ERR_UNSUPPORTED, "elemwise: %lld tiles", (long long)rowtiles);
        }
        if (dry) {
          if (red && groups > 1) {
            rc = reduce_final_pass(R, routp, rex, rexs, nullptr, ext_i, (int)groups, true, false);
            if (rc) return rc;
          }
          if (fused) *fused = red;
          return THX_OK;
        }
        const int64_t all_tiles = outer * tiles_t * tiles_i;
        int64_t grid = red ? groups * tiles_i : all_tiles;
        if (persist) {
          const int64_t cus = rt().ready ? rt().cus : 256;
          const int64_t per_cu = std::max<int64_t>(1, std::min<int64_t>(env_int("THX_EW_TR_BLOCKS_PER_CU", 8), (150 * 1024) / std::max<int64_t>(1, nbuf * lds_one)));
          grid = std::min(grid, cus * per_cu);
        }
        if (all_tiles * 256 <= 0xffffffffLL) {
          if (red && groups > 1) {
            rc = ensure_scratch((size_t)groups * ext_i * R->acc_bytes);
            if (rc) return rc;
          }
          ParamPack pk;
          for (int o = 0; o < nops; ++o) pk.put<char*>(views[o].ptr);
          for (int o = 0; o < nops; ++o) pk.put<uint64_t>(views[o].immval);
          pk.put<int32_t>((int32_t)ext_t);
          pk.put<int32_t>((int32_t)ext_i);
          pk.put<FastDivH>(make_fastdiv((uint64_t)tiles_i));
          pk.put<FastDivH>(make_fastdiv((uint64_t)tiles_t));
          for (int d = 0; d < ND; ++d) pk.put<FastDivH>(make_fastdiv(d < (int)odims.size() ? (uint64_t)dm.shape[odims[d]] : 1));
          for (int o = 0; o < nops; ++o)
            for (int d = 0; d < ND; ++d) pk.put<int32_t>(d < (int)odims.size() ? (int32_t)dm.stride[o][odims[d]] : 0);
          for (int o = 0; o < nops; ++o) pk.put<int32_t>((int32_t)dm.stride[o][tdim]);
          for (int o = 0; o < nops; ++o) pk.put<int32_t>((int32_t)dm.stride[o][ND - 1]);
          pk.align(8);
          if (!red) {
            pk.put<uint32_t>((uint32_t)all_tiles);
            pk.align(8);
          }
          if (red) {
            for (char* q : routp) pk.put<char*>(q);
            pk.put<uint64_t>(0);   // no further operands of the epilogue
            pk.put<int64_t>(1);
            pk.put<char*>(groups > 1 ? rt().scratch : nullptr);
            pk.put<int32_t>((int32_t)rowtiles);
            pk.put<int32_t>((int32_t)groups);
            pk.align(8);
          }
          rc = launch(k, e->name + "|" + plan, (unsigned)grid, block, pk.buf.data(), pk.buf.size());
          if (rc) return rc;
          if (red && groups > 1) {
            rc = reduce_final_pass(R, routp, rex, rexs, rt().scratch, ext_i, (int)groups, false, false);
            if (rc) return rc;
          }
          if (fused) *fused = red;
          return THX_OK;
        }
      }
    }
  }

  if (red_outs && e->red)   // the caller reduces the stored results next: they stay cacheable
    for (int w : e->red_of) views[e->n_in + w].reused = true;
  const int64_t nvec = ND == 1 ? n / vec : (n / inner) * row_vecs;
  // One vector per operand and thread: measured with inputs that are not cached, a larger unroll
  // never gains and costs registers (a seven-input float16 kernel needs 164 VGPRs at 4).
  int unr = 1;
  const int force_unr = env_int("THX_EW_UNR", 0);
  if (force_unr > 0) unr = force_unr;
  int block = 256;
  const int force_block = env_int("THX_EW_BLOCK", 0);
  if (force_block == 128 || force_block == 512 || force_block == 1024) block = force_block;
  const uint64_t nt = nt_mask(nt_streaming(moved), views);
  // grid-stride: a bounded number of blocks walk the index space instead of one block per chunk;
  // needed once one block per chunk would exceed the 2^32 - 1 work-items a dispatch can carry
  int gs = env_int("THX_EW_GS", 0);
  if (!gs && ceil_div64(nvec, (int64_t)block * unr) * block > 0xffffffffLL) gs = 64;

  // per operand and dimension: is the stride 0, 1 or anything; and which earlier operand has the
  // very same strides (its offset is reused)
  std::vector<std::vector<int>> sclass(nops, std::vector<int>(ND, 2));
  std::vector<int> alias(nops);
  std::string skey;
  for (int o = 0; o < nops; ++o) {
    alias[o] = o;
    for (int d = 0; d < ND; ++d) {
      const int64_t st = views[o].imm ? 0 : dm.stride[o][d];
      sclass[o][d] = st == 0 ? 0 : (st == 1 ? 1 : 2);
    }
    for (int q = 0; q < o && alias[o] == o; ++q)
      if (!views[o].imm && !views[q].imm &&
          std::equal(dm.stride[q].begin(), dm.stride[q].begin() + ND, dm.stride[o].begin()))
        alias[o] = q;
    for (int d = 0; d < ND; ++d) skey += char('0' + sclass[o][d]);
    if (alias[o] != o) skey += "a" + std::to_string(alias[o]);
    if (o + 1 < nops) skey += ".";
  }
  std::ostringstream key;
  key << "ew|nd" << ND << (wide ? "|i64" : "|i32") << "|v" << vec << "|u" << unr << "|s" << skey;
  if (nt) key << "|nt" << std::hex << nt << std::dec;
  key << (block != 256 ? "|b" + std::to_string(block) : "") << (gs ? "|gs" : "") << (ua ? "|ua" : "") << (rag ? "|rg" : "") << "|m";
  for (int o = 0; o < nops; ++o) key << mode[o] << (o + 1 < nops ? "," : "");
  const std::string plan = key.str() + (fast_div() ? "|fd" : "");
  set_last_plan(e->name + "|" + plan);

  Kernel k;
  auto it = e->plans.find(plan);
  if (it != e->plans.end() && (it->second.func || dry)) {
    k = it->second;
  } else {
    const std::string entry = entry_name(e->name, plan);
    std::ostringstream s;
    s << device_prelude() << e->src << "\nstruct ThxPlan {\n  typedef " << (wide ? "long long" : "int")
      << " IT;\n  enum { ND = " << ND << ", VEC = " << vec << ", UNR = " << unr << ", BLOCK = " << block
      << ", GS = " << (gs ? 1 : 0) << ", UA = " << ua << ", RAG = " << rag << " };\n  static constexpr unsigned long long NT = " << nt << "ull;\n  static constexpr int mode(int i) {\n    constexpr int m[] = {";
    for (int o = 0; o < nops; ++o) s << mode[o] << (o + 1 < nops ? ", " : "");
    s << "};\n    return m[i];\n  }\n  static constexpr int sclass(int i, int d) {\n    constexpr int m[][" << ND << "] = {";
    for (int o = 0; o < nops; ++o) {
      s << "{";
      for (int d = 0; d < ND; ++d) s << sclass[o][d] << (d + 1 < ND ? ", " : "");
      s << "}" << (o + 1 < nops ? ", " : "");
    }
    s << "};\n    return m[i][d];\n  }\n  static constexpr int alias(int i) {\n    constexpr int m[] = {";
    for (int o = 0; o < nops; ++o) s << alias[o] << (o + 1 < nops ? ", " : "");
    s << "};\n    return m[i];\n  }\n};\n"
      << "extern \"C\" __global__ __launch_bounds__(" << block << ") void " << entry << "(thx::EwParams<" << e->name
      << "::NOPS, ThxPlan::ND, ThxPlan::IT> p) {\n  thx::ew_body<" << e->name << ", ThxPlan>(p);\n}\n";
    rc = get_kernel(s.str(), entry, &k);
    if (rc) return rc;
    e->plans[plan] = k;
  }
  if (dry) return THX_OK;

  ParamPack pk;
  for (int o = 0; o < nops; ++o) pk.put<char*>(views[o].ptr);
  for (int o = 0; o < nops; ++o) pk.put<uint64_t>(views[o].immval);
  pk.put<int64_t>(nvec);
  pk.put<int64_t>(n);
  for (int d = 0; d < ND; ++d) {
    FastDivH f = make_fastdiv(d == ND - 1 && ND > 1 ? (uint64_t)row_vecs : (uint64_t)dm.shape[d]);
    if (d == ND - 1 && ND > 1) f.pad = (uint32_t)(inner - (row_vecs - 1) * vec);   // elements in a row's last vector
    pk.put<FastDivH>(f);
  }
  for (int o = 0; o < nops; ++o)
    for (int d = 0; d < ND; ++d) pk.put_index(wide, dm.stride[o][d]);
  pk.align(8);

  int64_t grid = (nvec + (int64_t)block * unr - 1) / ((int64_t)block * unr);
  if (grid < 1) grid = 1;
  if (gs) grid = std::min<int64_t>(grid, (int64_t)(rt().ready ? rt().cus : 256) * gs);
  if (grid * block > 0xffffffffLL)
    return fail(THX_ERR_UNSUPPORTED, "elemwise: %lld blocks of %d exceed the work-items of one dispatch", (long long)grid, block);
  return launch(k, e->name + "|" + plan, (unsigned)grid, block, pk.buf.data(), pk.buf.size());
}

extern "C" {

int thx_elemwise_call(thx_elemwise* e, const thx_array* ins, const thx_array* outs, int flags) {
  return elemwise_impl(e, ins, outs, nullptr, flags, nullptr);
}

int thx_elemwise_attach_reduce(thx_elemwise* e, thx_reduce* r, const int32_t* which_outputs) {
  if (!e) return fail(THX_ERR_ARG, "thx_elemwise_attach_reduce: null argument");
  if (!r) {   // detach: `e` no longer refers to the reduction, which may now be freed first
    e->red = nullptr;
    e->red_of.clear();
    return THX_OK;
  }
  if (!which_outputs) return fail(THX_ERR_ARG, "thx_elemwise_attach_reduce: null argument");
  if (r->n_extra) return fail(THX_ERR_UNSUPPORTED, "thx_elemwise_attach_reduce: the reduction's epilogue may take no further operands");
  for (int i = 0; i < r->n_in; ++i) {
    const int w = which_outputs[i];
    if (w < 0 || w >= e->n_out) return fail(THX_ERR_ARG, "thx_elemwise_attach_reduce: output %d of %d", w, e->n_out);
    if (r->dtypes[i] != e->dtypes[e->n_in + w])
      return fail(THX_ERR_TYPE, "thx_elemwise_attach_reduce: the reduction reads dtype code %d, output %d has %d",
                  r->dtypes[i], w, e->dtypes[e->n_in + w]);
  }
  e->red = r;
  e->red_of.assign(which_outputs, which_outputs + r->n_in);
  return THX_OK;
}

int thx_elemwise_reduce_call(thx_elemwise* e, const thx_array* ins, const thx_array* outs, const thx_array* red_outs,
                             int flags) {
  if (!e || !red_outs) return fail(THX_ERR_ARG, "thx_elemwise_reduce_call: null argument");
  if (!e->red) return fail(THX_ERR_ARG, "thx_elemwise_reduce_call: no reduction is attached to this operation");
  bool fused = false;
  int rc = elemwise_impl(e, ins, outs, red_outs, flags, &fused);
  if (rc || fused) return rc;
  // any other plan: the stored results are reduced over every dimension but the last
  thx_reduce* r = e->red;
  const int nd = outs[0].nd;
  if (nd < 1) return fail(THX_ERR_TYPE, "thx_elemwise_reduce_call: results of rank 0 have nothing to reduce");
  std::vector<thx_array> rin(r->n_in);
  for (int i = 0; i < r->n_in; ++i) {
    rin[i] = outs[e->red_of[i]];
  }
  uint8_t mask[THX_MAX_ND];
  for (int d = 0; d < nd; ++d) mask[d] = d < nd - 1;
  const std::string plan = thx_last_plan();
  rc = thx_reduce_call(r, rin.data(), mask, red_outs, flags);
  if (!rc) set_last_plan(plan + " + " + thx_last_plan());
  return rc;
}

}  // extern "C"
