// Reduction planner: canonicalises (shape, strides, mask) into kept and reduced
// dimension lists, chooses the row, column or generic kernel form, sizes the
// slice split for the device, compiles on first use and launches one or two
// passes.
#include <algorithm>
#include <array>
#include <cstdlib>
#include <cstring>
#include <sstream>
#include <unordered_map>

#include "thx_internal.h"

namespace thx {

enum { M_VEC = 0, M_BCAST = 1, M_GATHER = 2, M_IMM = 3, M_IOTA = 4 };

struct Dim {
  int64_t extent;
  std::vector<int64_t> stride;  // per input
};

static void merge_dims(std::vector<Dim>* v) {
  std::vector<Dim> out;
  for (const Dim& d : *v) {
    if (!out.empty()) {
      Dim& o = out.back();  // o is the outer neighbour of d
      bool ok = true;
      for (size_t i = 0; i < d.stride.size() && ok; ++i) ok = o.stride[i] == d.stride[i] * d.extent;
      if (ok) {
        o.extent *= d.extent;
        o.stride = d.stride;
        continue;
      }
    }
    out.push_back(d);
  }
  v->swap(out);
}

static int64_t iabs(int64_t x) { return x < 0 ? -x : x; }
static int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }
static int64_t round_up(int64_t a, int64_t b) { return ceil_div(a, b) * b; }
static int env_int(const char* name, int dflt) {
  const char* v = getenv(name);
  return v ? atoi(v) : dflt;
}

static std::string plan_struct(bool wide, const std::vector<std::pair<std::string, int64_t>>& consts,
                               const std::vector<int>& mode, uint64_t nt,
                               const std::vector<std::array<int, 2>>& sclass = {}) {
  std::ostringstream s;
  s << "\nstruct ThxPlan {\n  typedef " << (wide ? "long long" : "int") << " IT;\n  enum { ";
  for (size_t i = 0; i < consts.size(); ++i) s << consts[i].first << " = " << consts[i].second << (i + 1 < consts.size() ? ", " : "");
  s << " };\n  static constexpr unsigned long long NT = " << nt << "ull;\n  static constexpr int mode(int i) {\n    constexpr int m[] = {";
  for (size_t i = 0; i < mode.size(); ++i) s << mode[i] << (i + 1 < mode.size() ? ", " : "");
  s << "};\n    return m[i];\n  }\n";
  if (!sclass.empty()) {
    s << "  static constexpr int sclass(int i, int w) {\n    constexpr int m[][2] = {";
    for (size_t i = 0; i < sclass.size(); ++i)
      s << "{" << sclass[i][0] << ", " << sclass[i][1] << "}" << (i + 1 < sclass.size() ? ", " : "");
    s << "};\n    return m[i][w];\n  }\n";
  }
  s << "};\n";
  return s.str();
}

static int final_tpo(int64_t n_out) { return n_out >= 1024 ? 1 : (n_out >= 16 ? 64 : 256); }

// The message of a call that may neither compile nor load a kernel and finds the one it needs missing.
static int not_loaded(const thx_reduce* r, const std::string& plan) {
  return fail(THX_ERR_UNSUPPORTED,
              "thx_reduce_call_static: kernel '%s|%s' is not loaded; loading one allocates device memory, so run "
              "thx_reduce_call once on operands of this layout first", r->name.c_str(), plan.c_str());
}

// `fixed`: the call comes from thx_reduce_call_static - only kernels that are already loaded, no events.
int reduce_final_pass(thx_reduce* r, const std::vector<char*>& outp, const std::vector<uint64_t>& ex,
                      const std::vector<int64_t>& exs, char* partial, int64_t n_out, int S, bool dry, bool fixed) {
  const int tpo = final_tpo(n_out);
  const std::string plan = "rf|t" + std::to_string(tpo);
  Kernel k;
  auto it = r->plans.find(plan);
  if (it != r->plans.end() && (it->second.func || dry)) {
    k = it->second;
  } else if (fixed) {
    return not_loaded(r, plan);
  } else {
    const std::string entry = entry_name(r->name, plan);
    std::ostringstream s;
    s << device_prelude() << r->src << "\nextern \"C\" __global__ __launch_bounds__(256) void " << entry << "(thx::FinalParams<"
      << r->name << "::NOUT, " << r->name << "::NEX> p) {\n  thx::red_final_body<" << r->name << ", 256, " << tpo << ">(p);\n}\n";
    int rc = get_kernel(s.str(), entry, &k);
    if (rc) return rc;
    r->plans[plan] = k;
  }
  if (dry) return THX_OK;
  ParamPack pk;
  for (char* p : outp) pk.put<char*>(p);
  for (uint64_t v : ex) pk.put<uint64_t>(v);
  for (int64_t v : exs) pk.put<int64_t>(v);
  pk.put<char*>(partial);
  pk.put<int64_t>(n_out);
  pk.put<int32_t>(S);
  pk.put<int32_t>(0);
  pk.align(8);
  const int64_t grid = ceil_div(n_out, 256 / tpo);
  if (grid * 256 > 0xffffffffLL)   // a reduction is only split when it has few outputs
    return fail(THX_ERR_UNSUPPORTED, "reduce: second pass over %lld outputs", (long long)n_out);
  return launch(k, r->name + "|" + plan, (unsigned)grid, 256, pk.buf.data(), pk.buf.size(), fixed);
}

// Where the partial results of a split reduction go: the buffer the library allocates and grows
// (thx_reduce_call), or the fixed array (thx_reduce_call_static), which cannot grow.  In the fixed
// case the second pass's kernel is looked up here too, so that a miss is reported before the
// first pass is launched.
static int partial_buffer(thx_reduce* r, size_t bytes, int64_t n_out, bool fixed, char** out) {
  if (!fixed) {
    int rc = ensure_scratch(bytes);
    if (rc) return rc;
    *out = rt().scratch;
    return THX_OK;
  }
  if (bytes > (size_t)THX_STATIC_SCRATCH_BYTES)
    return fail(THX_ERR_UNSUPPORTED,
                "thx_reduce_call_static: this reduction needs %zu bytes of partial results, the fixed scratch array "
                "holds %zu; use thx_reduce_call", bytes, (size_t)THX_STATIC_SCRATCH_BYTES);
  const std::string fplan = "rf|t" + std::to_string(final_tpo(n_out));
  auto it = r->plans.find(fplan);
  if (it == r->plans.end() || !it->second.func) return not_loaded(r, fplan);
  *out = rt().static_scratch;
  return THX_OK;
}

}  // namespace thx

using namespace thx;

extern "C" {

int thx_reduce_new(const char* functor_src, const char* functor_name, int n_in, int n_out, int n_extra,
                   const int32_t* dtypes, int acc_bytes, thx_reduce** out) {
  if (!functor_src || !functor_name || !dtypes || !out) return fail(THX_ERR_ARG, "thx_reduce_new: null argument");
  if (n_in < 1 || n_out < 1 || n_extra < 0 || acc_bytes < 1)
    return fail(THX_ERR_ARG, "thx_reduce_new: needs inputs, outputs and an accumulator");
  for (int i = 0; i < n_in + n_out + n_extra; ++i)
    if (!dtype_size(dtypes[i])) return fail(THX_ERR_TYPE, "thx_reduce_new: unknown dtype code %d", dtypes[i]);
  thx_reduce* r = new thx_reduce;
  r->src = functor_src;
  r->name = functor_name;
  r->n_in = n_in;
  r->n_out = n_out;
  r->n_extra = n_extra;
  r->acc_bytes = acc_bytes;
  r->dtypes.assign(dtypes, dtypes + n_in + n_out + n_extra);
  r->has_ticket = r->src.find("ticket_pack") != std::string::npos;
  *out = r;
  return THX_OK;
}

int thx_reduce_free(thx_reduce* r) {
  delete r;
  return THX_OK;
}

}  // extern "C"

// Both entry points.  `fixed` (thx_reduce_call_static): partial results go to the library's fixed
// scratch array, and nothing on the way may allocate device memory - no hipMalloc / hipFree, no
// compilation or module load (a kernel that is not loaded yet is an error), no event creation.
static int reduce_impl(thx_reduce* r, const thx_array* ins, const uint8_t* reduce_mask, const thx_array* outs, int flags,
                       bool fixed) {
  if (!r || !ins || !outs) return fail(THX_ERR_ARG, "thx_reduce_call: null argument");
  const bool dry = (flags & THX_DRY_RUN) != 0;
  if (fixed) {
    if (dry) return fail(THX_ERR_ARG, "thx_reduce_call_static: THX_DRY_RUN is for thx_reduce_call");
    if (!rt().ready || !rt().static_scratch)
      return fail(THX_ERR_ARG, "thx_reduce_call_static: call thx_init first (it resolves the scratch array's address)");
  } else if (!dry) {
    int rc = ensure_init();
    if (rc) return rc;
  }
  const int NIN = r->n_in, NOUT = r->n_out;
  int nd = 0;
  int64_t shape[THX_MAX_ND];
  std::vector<View> views;
  int rc = gather_inputs("reduce", ins, NIN, r->dtypes.data(), flags, &nd, shape, &views);
  if (rc) return rc;
  if (nd > 0 && !reduce_mask) return fail(THX_ERR_ARG, "thx_reduce_call: null mask");
  // THX_INDEX operands: the element's position within the reduced dimensions, in C order
  for (int i = 0; i < NIN; ++i) {
    if (!(ins[i].dtype & THX_INDEX)) continue;
    View& v = views[i];
    v.iota = true;
    v.ptr = nullptr;
    int64_t mult = 1;
    for (int d = nd - 1; d >= 0; --d) {
      v.stride[d] = reduce_mask[d] ? mult : 0;
      if (reduce_mask[d]) mult *= shape[d];
    }
  }
  // outputs: C-contiguous arrays of the kept dimensions
  int64_t kshape[THX_MAX_ND];
  int nk_full = 0;
  int64_t n_out = 1, n_red = 1;
  for (int d = 0; d < nd; ++d) {
    if (reduce_mask[d]) {
      n_red *= shape[d];
    } else {
      kshape[nk_full++] = shape[d];
      n_out *= shape[d];
    }
  }
  std::vector<char*> outp(NOUT);
  for (int o = 0; o < NOUT; ++o) {
    const thx_array& a = outs[o];
    if (a.nd != nk_full) return fail(THX_ERR_TYPE, "reduce: output %d has rank %d, expected %d", o, a.nd, nk_full);
    const int adt = a.dtype & ~THX_REUSED;   // results are small: the hint changes nothing for them
    if (adt != r->dtypes[NIN + o])
      return fail(THX_ERR_TYPE, "reduce: output %d has dtype code %d, the operation was built for %d", o, adt,
                  r->dtypes[NIN + o]);
    const int isz = dtype_size(adt);
    int64_t expect = isz;
    for (int d = nk_full - 1; d >= 0; --d) {
      if (a.shape[d] != kshape[d])
        return fail(THX_ERR_SHAPE, "reduce: output %d has extent %lld along dimension %d, the result has %lld", o,
                    (long long)a.shape[d], d, (long long)kshape[d]);
      // an array without elements has no layout to speak of (its strides depend on who computed them)
      if (n_out > 0 && a.shape[d] > 1 && a.strides_bytes[d] != expect)
        return fail(THX_ERR_TYPE, "reduce: output %d is not C-contiguous", o);
      expect *= a.shape[d];
    }
    if (null_base(a, dry)) return fail(THX_ERR_ARG, "reduce: output %d has no base address", o);
    outp[o] = (char*)a.base + a.offset_bytes;
    if (((uintptr_t)outp[o]) % isz) return fail(THX_ERR_TYPE, "reduce: output %d is not aligned to its element size", o);
  }
  // Operands of the epilogue follow the reduced inputs: a host scalar is passed by value; a device
  // array holds one value per result (the results' element count) and is passed by address and element
  // stride, the epilogue reads it at the result's index times that stride.  Its layout must be that of a
  // C-contiguous array with every stride scaled by one factor (a contiguous array, or a view that keeps
  // the results' dimensions in order, such as x[0, :, 0, 0]).
  std::vector<uint64_t> ex(std::max(1, r->n_extra), 0);
  std::vector<int64_t> exs(std::max(1, r->n_extra), 1);
  for (int j = 0; j < r->n_extra; ++j) {
    const thx_array& a = ins[NIN + j];
    const int want = r->dtypes[NIN + NOUT + j];
    if ((a.dtype & ~(THX_HOST_SCALAR | THX_REUSED)) != want)
      return fail(THX_ERR_TYPE, "reduce: epilogue operand %d has dtype code %d, the operation was built for %d", j,
                  a.dtype & ~(THX_HOST_SCALAR | THX_REUSED), want);
    if (null_base(a, dry)) return fail(THX_ERR_ARG, "reduce: epilogue operand %d has no base address", j);
    const char* p = (const char*)a.base + a.offset_bytes;
    if (a.dtype & THX_HOST_SCALAR) {
      if (dtype_size(want) > 8)
        return fail(THX_ERR_TYPE, "reduce: epilogue operand %d: values of %d bytes do not travel by value", j, dtype_size(want));
      memcpy(&ex[j], p, (size_t)dtype_size(want));
      continue;
    }
    const int64_t isz = dtype_size(want);
    int64_t count = 1, expect = 0;
    for (int d = a.nd - 1; d >= 0; --d) count *= a.shape[d];
    const bool has_elements = count > 0;
    count = 1;
    for (int d = a.nd - 1; d >= 0; --d) {
      if (a.shape[d] > 1 && has_elements) {
        if (!expect) {
          if (a.strides_bytes[d] % isz || !a.strides_bytes[d])
            return fail(THX_ERR_TYPE, "reduce: epilogue operand %d has a stride that is not a multiple of its element size", j);
          expect = a.strides_bytes[d];
          exs[j] = a.strides_bytes[d] / isz;
        }
        if (a.strides_bytes[d] != expect)
          return fail(THX_ERR_TYPE, "reduce: epilogue operand %d is not laid out like a C-contiguous array", j);
        expect *= a.shape[d];
      }
      count *= a.shape[d];
    }
    if (count != n_out)
      return fail(THX_ERR_SHAPE, "Input dimension mis-match. (epilogue operand %d has %lld elements, the result has %lld)",
                  j, (long long)count, (long long)n_out);
    if (((uintptr_t)p) % isz)
      return fail(THX_ERR_TYPE, "reduce: epilogue operand %d is not aligned to its element size", j);
    ex[j] = (uint64_t)(uintptr_t)p;
  }
  if (n_out == 0) {
    set_last_plan("red|empty");
    return THX_OK;
  }
  if (n_red == 0) {  // identity through the epilogue
    set_last_plan(r->name + "|rf|identity");
    return reduce_final_pass(r, outp, ex, exs, nullptr, n_out, 0, dry, fixed);
  }

  // primary input: the one that spans the most memory
  int primary = 0;
  {
    int64_t best = -1;
    for (int i = 0; i < NIN; ++i) {
      if (views[i].iota) continue;
      int64_t foot = 1;
      for (int d = 0; d < nd; ++d)
        if (views[i].stride[d] != 0) foot *= shape[d];
      foot *= dtype_size(views[i].dtype);
      if (foot > best) {
        best = foot;
        primary = i;
      }
    }
  }
  std::vector<Dim> KD, RD;
  for (int d = 0; d < nd; ++d) {
    if (shape[d] == 1) continue;
    Dim dm;
    dm.extent = shape[d];
    for (int i = 0; i < NIN; ++i) dm.stride.push_back(views[i].stride[d]);
    (reduce_mask[d] ? RD : KD).push_back(dm);
  }
  // reduced dimensions commute: walk them from the largest stride to the smallest
  std::stable_sort(RD.begin(), RD.end(),
                   [&](const Dim& a, const Dim& b) { return iabs(a.stride[primary]) > iabs(b.stride[primary]); });
  merge_dims(&KD);
  merge_dims(&RD);
  // Nothing left to reduce - every reduced extent is 1, a copy through the accumulator and the epilogue: as the one
  // "row" of the column form its elements are read and written as vectors (one element per thread otherwise,
  // 1.5 TB/s of input for 256 MB of float32).
  if (RD.empty() && !KD.empty() && KD.back().stride[primary] == 1 && KD.back().extent >= 1024 && env_int("THX_RED_COPY_AS_COL", 1)) {
    Dim one;
    one.extent = 1;
    one.stride.assign(NIN, 0);
    RD.push_back(one);
  }
  const int NKD = (int)KD.size(), NR = (int)RD.size();

  const int cus = rt().ready ? rt().cus : 256;
  // blocks wanted when a reduction has to be split to fill the device: few, so that the second pass stays tiny
  const int bpc = env_int("THX_RED_BLOCKS_PER_CU", 0);
  // A reduction that carries positions (argmax) spends several times the instructions of a sum on each element:
  // with one block on a compute unit nothing covers its arithmetic while loads are in flight, so the column form
  // asks for two blocks a unit and keeps fewer rows in flight per thread (measured on the (8192, 8192) float32
  // argmax over axis 0: 45.0 us against 52.6 us).
  bool carries_positions = false;
  for (int i = 0; i < NIN; ++i) carries_positions = carries_positions || views[i].iota;
  const int64_t target_row = (int64_t)cus * (bpc > 0 ? bpc : 2);
  const int64_t target_col = (int64_t)cus * (bpc > 0 ? bpc : (carries_positions ? 2 : 1));

  bool wide = n_out >= (int64_t(1) << 31) - 65536 || n_red >= (int64_t(1) << 31) - 65536;
  for (int i = 0; i < NIN && !wide; ++i) {
    int64_t span = 0;
    for (const Dim& d : KD) span += (d.extent - 1) * iabs(d.stride[i]);
    for (const Dim& d : RD) span += (d.extent - 1) * iabs(d.stride[i]);
    if (span >= (int64_t(1) << 31) - 65536) wide = true;
  }

  enum { ROW, COL, GEN, STRIP } form;
  if (NR > 2) form = GEN;
  else if (NR == 0 || NKD == 0) form = ROW;
  else if (iabs(RD.back().stride[primary]) == 1) form = ROW;
  else if (KD.back().stride[primary] == 1) form = COL;
  else form = ROW;
  // the column form counts columns in 32 bits
  if (form == COL && KD.back().extent >= (int64_t(1) << 31) - 65536) form = GEN;
  // The column form gives every block of 256 threads one strip of at most 64 column vectors and spreads the
  // rows over the remaining lanes: with few columns and few rows (sums over a middle axis of extent 4 of a
  // (n, 4, 4, 4) array) nearly all of them idle - 17 to 290 GB/s measured.  One thread per result, which the
  // generic form is, reads such an array at memory speed: neighbouring results lie next to each other.
  if (form == COL && KD.back().extent < 64 && n_red * 4 <= 256 / std::max<int64_t>(1, std::min<int64_t>(64, KD.back().extent)))
    form = GEN;
  // Two to four rows of columns that cannot be read as vectors - an odd extent or an unaligned view, and too few
  // columns for element-aligned vectors: one thread per result (with 4-byte accesses a (3, 22369621) float32 sum over
  // axis 0 ran at 1.2 TB/s in the column form against 2.6 TB/s; with 16-byte accesses, aligned or not, the column
  // form is the faster one: 2.9 TB/s for three rows, 3.9 against 2.8 for four).
  if (form == COL && n_red <= 4) {
    bool vectors = KD.back().extent % 2 == 0;
    for (int i = 0; i < NIN && vectors; ++i) {
      if (views[i].iota || views[i].imm || KD.back().stride[i] != 1) continue;
      const size_t two = (size_t)dtype_size(views[i].dtype) * 2;
      if (((uintptr_t)views[i].ptr) % two) vectors = false;
      for (const Dim& d : RD)
        if (d.stride[i] % 2) vectors = false;
      for (size_t d = 0; d + 1 < KD.size(); ++d)
        if (KD[d].stride[i] % 2) vectors = false;
    }
    // ... unless the column form can read them as element-aligned vectors
    int maxsz = 0;
    for (int i = 0; i < NIN; ++i)
      if (!views[i].iota && !views[i].imm && KD.back().stride[i] == 1) maxsz = std::max(maxsz, dtype_size(views[i].dtype));
    const bool unaligned_vectors = env_int("THX_RED_UA", 1) && maxsz && KD.back().extent >= (int64_t)(16 / maxsz) * env_int("THX_RED_UA_MINVEC", 4);
    if (!vectors && !unaligned_vectors) form = GEN;
  }
  // A C-contiguous (rows, C) array with at most 16 columns, fewer than four vectors hold, reduced over its many rows
  // ((22 369 621, 3) float32: 2.6 TB/s with 4 threads across a strip of columns; float16: 1.4): walked as the flat
  // run of elements it is.
  int strip_vec = 0;
  if ((form == COL || form == GEN) && NKD == 1 && NR == 1 && env_int("THX_RED_STRIP", 1)) {
    const int64_t C = KD[0].extent, rows = RD[0].extent;
    int maxsz = 0;
    bool ok = C >= 2 && C <= 16 && rows * C >= (int64_t(1) << 16) && C * (int64_t)r->acc_bytes <= 256;   // accumulators of one thread; 256 times as much LDS
    for (int i = 0; i < NIN && ok; ++i) {
      if (views[i].imm) continue;
      if (views[i].iota || KD[0].stride[i] != 1 || RD[0].stride[i] != C) ok = false;
      if (((uintptr_t)views[i].ptr) % (size_t)dtype_size(views[i].dtype)) ok = false;
      maxsz = std::max(maxsz, dtype_size(views[i].dtype));
    }
    // two or more whole vectors of columns are as well off in the column form (float16, 16 columns: 5.6 against 4.5 TB/s)
    if (ok && maxsz && maxsz <= 8 && C < (int64_t)(16 / maxsz) * 4 && !(C % (16 / maxsz) == 0 && C / (16 / maxsz) >= 2)) {
      form = STRIP;
      strip_vec = 16 / maxsz;
    }
  }
  const char* force = getenv("THX_RED_FORM");
  if (force && NR <= 2 && NR > 0) {
    if (!strcmp(force, "row")) form = ROW;
    if (!strcmp(force, "col") && NKD > 0 && KD.back().extent < (int64_t(1) << 31) - 65536) form = COL;
    if (!strcmp(force, "gen")) form = GEN;
  }

  auto vec_width = [&](const std::vector<int>& mode) {
    int maxsz = 0;
    for (int i = 0; i < NIN; ++i)
      if (mode[i] == M_VEC) maxsz = std::max(maxsz, dtype_size(views[i].dtype));
    return maxsz ? 16 / maxsz : 1;
  };

  const int block = 256;
  const uint64_t nt = nt_mask(nt_choice(1), views);  // a reduction streams whatever nothing reads again
  std::string plan;
  Kernel k;
  ParamPack pk;
  int64_t nblocks = 0;     // pieces of work: (block of outputs) x (slice of the reduce domain)
  bool gs = false;         // more pieces than one dispatch holds blocks
  const int forced_limit = env_int("THX_RED_MAX_DISPATCH", 0);   // a smaller limit, to exercise the striding kernels
  const int64_t max_dispatch = forced_limit >= 1024 ? forced_limit : 0xffffffffLL;
  int S = 1;
  int launch_block = block;
  char* partial = nullptr;  // Acc[S][n_out] of a split reduction
  bool one_launch = false;  // the slices settle the result among themselves (ticket_finish)

  if (form == ROW) {
    const int64_t RC = NR ? RD.back().extent : 1;
    const int64_t RA = NR == 2 ? RD[0].extent : 1;
    const int ra2 = NR == 2;
    std::vector<int> mode(NIN);
    std::vector<int64_t> rc_stride(NIN), ra_stride(NIN);
    for (int i = 0; i < NIN; ++i) {
      rc_stride[i] = NR ? RD.back().stride[i] : 0;
      ra_stride[i] = ra2 ? RD[0].stride[i] : 0;
      mode[i] = rc_stride[i] == 1 ? M_VEC : (rc_stride[i] == 0 ? M_BCAST : M_GATHER);
      if (views[i].imm) mode[i] = M_IMM;
      if (views[i].iota) mode[i] = M_IOTA;
    }
    int vec = vec_width(mode);
    auto vec_ok = [&](int v) {
      if (v == 1) return true;
      if (RC % v) return false;
      if (ra2 && RC / v < 2) return false;
      for (int i = 0; i < NIN; ++i) {
        if (mode[i] != M_VEC) continue;
        if (((uintptr_t)views[i].ptr) % (size_t)(dtype_size(views[i].dtype) * v)) return false;
        if (ra_stride[i] % v) return false;
        for (const Dim& d : KD)
          if (d.stride[i] % v) return false;
      }
      return true;
    };
    const int vec_full = vec;
    while (!vec_ok(vec)) vec /= 2;
    // Rows that are long but of a length that is no multiple of the vector width, or that do not start on a vector
    // boundary (a sum of all 134 217 727 float16 elements of an array read 2 bytes per lane: 1.8 TB/s; int8: 0.75):
    // full-width vectors through element-aligned pointers, and the last RC mod vec elements of a row one by one.
    int ua = 0;
    if (vec < vec_full && !ra2 && NR == 1 && RC >= (int64_t)vec_full * 16 && env_int("THX_RED_UA", 1)) {
      bool ok = true;
      for (int i = 0; i < NIN; ++i)
        if (mode[i] == M_VEC && ((uintptr_t)views[i].ptr) % (size_t)dtype_size(views[i].dtype)) ok = false;
      if (ok) {
        vec = vec_full;
        ua = 1;
      }
    }
    const int64_t nvec = RA * RC / vec;
    int tpr = nvec >= 512 ? 256 : nvec >= 64 ? 64 : nvec >= 16 ? 16 : nvec >= 4 ? 4 : 1;
    const int force_tpr = env_int("THX_RED_TPR", 0);
    if (force_tpr > 0 && force_tpr <= 256 && (force_tpr & (force_tpr - 1)) == 0) tpr = force_tpr;
    const int64_t per_thread = ceil_div(nvec, tpr);
    int unr = per_thread >= 4 ? 4 : per_thread >= 2 ? 2 : 1;
    const int force_unr = env_int("THX_RED_UNR", 0);
    if (force_unr > 0) unr = force_unr;
    int nacc = unr;  // accumulator sets per thread
    // few outputs, long reduce domains: 1024 threads per output before resorting to a split
    int rblock = block;
    if (tpr == 256 && env_int("THX_RED_BIGBLOCK", 1) && ceil_div(n_out, 1) * 2 <= target_row * 4 &&
        n_out >= cus / 2 && nvec >= 1024 * 8) {
      rblock = 1024;
      tpr = 1024;
    }
    const bool bigblock = rblock == 1024;
    // One 1024-thread block per result with several full-sized operands (batch-norm gradient statistics over
    // x and g): two vectors per operand in flight per thread measured 1 - 2 us faster than four on 205 MB
    // (39.6 against 40.8 us; one operand alone is indifferent, 19.6 - 19.8 us on 103 MB)
    {
      int n_vec = 0;
      for (int i = 0; i < NIN; ++i) n_vec += mode[i] == M_VEC;
      if (bigblock && ra2 && n_vec >= 2 && unr > 2 && force_unr <= 0) unr = 2;
      if (nacc > unr) nacc = unr;
    }
    // a split reduction of one (or very few) results with larger blocks: fewer slices for the same number of waves
    const int split_threads = env_int("THX_RED_SPLIT_THREADS", 0);
    if (!bigblock && tpr == 256 && (split_threads == 512 || split_threads == 1024) && n_out * 2 <= target_row)
      rblock = tpr = split_threads;
    // Slices that settle the result with one atomic add each (any / all) queue up on one word: few, large
    // slices - one block of 1024 threads per compute unit - keep that queue short (19.2 us against 21.8 us
    // with two blocks of 256 per unit for the (64, 128, 56, 56) int32 any + all; 20.5 us with a second launch).
    int64_t want_blocks = target_row;
    if (!bigblock && tpr == 256 && !split_threads && r->has_ticket && n_out <= THX_TICKET_WORDS && n_out * 2 <= cus &&
        env_int("THX_RED_TICKET", 1) && !bpc) {
      rblock = tpr = 1024;
      want_blocks = cus;
    }
    const int force_nacc = env_int("THX_RED_NACC", 0);
    if (force_nacc > 0) nacc = force_nacc;
    if (nacc > unr) nacc = unr;
    const int rpb = rblock / tpr;
    const int64_t oblocks = ceil_div(n_out, rpb);
    int64_t chunk = nvec;
    if (!bigblock && oblocks * 2 <= want_blocks && nvec >= (int64_t)tpr * unr * 4) {
      int64_t want = std::min(ceil_div(want_blocks, oblocks), nvec / ((int64_t)tpr * unr * 2));
      if (want > 1) {
        chunk = round_up(ceil_div(nvec, want), (int64_t)tpr * unr);
        S = (int)ceil_div(nvec, chunk);
      }
    }
    if (ra2 && nvec >= (int64_t(1) << 31) - 65536) wide = true;
    const bool ticket = S > 1 && r->has_ticket && n_out <= THX_TICKET_WORDS && S < 65536 && env_int("THX_RED_TICKET", 1);
    one_launch = ticket;
    const int NK = std::max(1, NKD);
    std::vector<std::array<int, 2>> sclass(NIN);
    std::string skey;
    for (int i = 0; i < NIN; ++i) {
      auto cls = [](int64_t st) { return st == 0 ? 0 : (st == 1 ? 1 : 2); };
      sclass[i] = {views[i].imm ? 0 : cls(ra_stride[i]), views[i].imm ? 0 : cls(rc_stride[i])};
      skey += char('0' + sclass[i][0]);
      skey += char('0' + sclass[i][1]);
    }
    nblocks = oblocks * S;
    gs = nblocks * rblock > max_dispatch;
    // One 1024-thread block per result whose reduce domain is slabs around the kept axis: the slabs of
    // neighbouring results meet inside cache lines, so each die (blocks go to the eight dies in turn, one L2
    // each) takes a contiguous eighth of the results and fetches those lines once.
    const bool xcd = bigblock && ra2 && S == 1 && !gs && nblocks % 8 == 0 && env_int("THX_RED_XCD", 1);
    std::ostringstream key;
    key << "rr|k" << NK << (wide ? "|i64" : "|i32") << "|v" << vec << "|u" << unr << (nacc != unr ? "|c" + std::to_string(nacc) : "") << "|t" << tpr << "|a" << ra2 << "|s" << skey << (nt ? "|nt" + std::to_string(nt) : "") << (ticket ? "|tk" : "") << (gs ? "|gs" : "") << (xcd ? "|x8" : "") << (ua ? "|ua" : "") << "|m";
    for (int i = 0; i < NIN; ++i) key << mode[i] << (i + 1 < NIN ? "," : "");
    plan = key.str() + (fast_div() ? "|fd" : "");
    auto it = r->plans.find(plan);
    if (it != r->plans.end() && (it->second.func || dry)) {
      k = it->second;
    } else if (fixed) {
      return not_loaded(r, plan);
    } else {
      const std::string entry = entry_name(r->name, plan);
      std::ostringstream s;
      s << device_prelude() << r->src
        << plan_struct(wide, {{"NK", NK}, {"VEC", vec}, {"UNR", unr}, {"NACC", nacc}, {"BLOCK", rblock}, {"TPR", tpr}, {"RA2", ra2}, {"TICKET", ticket ? 1 : 0}, {"GS", gs ? 1 : 0}, {"XCD", xcd ? 1 : 0}, {"UA", ua}}, mode, nt, sclass)
        << "extern \"C\" __global__ __launch_bounds__(" << rblock << ") void " << entry << "(thx::RowParams<" << r->name
        << "::NIN, " << r->name << "::NOUT, " << r->name << "::NEX, ThxPlan::NK, ThxPlan::IT> p) {\n  thx::red_row_body<" << r->name
        << ", ThxPlan>(p);\n}\n";
      rc = get_kernel(s.str(), entry, &k);
      if (rc) return rc;
      r->plans[plan] = k;
    }
    if (!dry && S > 1) {
      if (ticket) {
        partial = rt().ticket_words;
      } else {
        rc = partial_buffer(r, (size_t)S * n_out * r->acc_bytes, n_out, fixed, &partial);
        if (rc) return rc;
      }
    }
    for (int i = 0; i < NIN; ++i) pk.put<char*>(views[i].ptr);
    for (int i = 0; i < NIN; ++i) pk.put<uint64_t>(views[i].immval);
    for (int o = 0; o < NOUT; ++o) pk.put<char*>(outp[o]);
    for (uint64_t v : ex) pk.put<uint64_t>(v);
    for (int64_t v : exs) pk.put<int64_t>(v);
    pk.put<char*>(partial);
    pk.put<int64_t>(n_out);
    pk.put<int64_t>(nblocks);
    pk.put<int64_t>(nvec);
    pk.put<int64_t>(chunk);
    pk.put<int64_t>(RC);
    pk.put<int32_t>(S);
    pk.put<int32_t>(0);
    for (int d = 0; d < NK; ++d) pk.put<FastDivH>(make_fastdiv(d < NKD ? (uint64_t)KD[d].extent : 1));
    pk.put<FastDivH>(make_fastdiv((uint64_t)std::max<int64_t>(1, RC / vec)));
    for (int i = 0; i < NIN; ++i)
      for (int d = 0; d < NK; ++d) pk.put_index(wide, d < NKD ? KD[d].stride[i] : 0);
    for (int i = 0; i < NIN; ++i) pk.put_index(wide, ra_stride[i]);
    for (int i = 0; i < NIN; ++i) pk.put_index(wide, rc_stride[i]);
    pk.align(8);
    launch_block = rblock;
  } else if (form == COL) {
    int cblock = block;   // threads per block of the column kernel
    const int force_cb = env_int("THX_RED_COLBLOCK", 0);
    if (force_cb == 256 || force_cb == 512 || force_cb == 1024) cblock = force_cb;
    const int64_t C = KD.back().extent;
    const int ko = NKD - 1;  // outer kept dimensions
    const int NK = std::max(1, ko);
    const int rr2 = NR == 2;
    const int64_t rows = n_red;
    std::vector<int> mode(NIN);
    std::vector<int64_t> c_stride(NIN), r0_stride(NIN), r1_stride(NIN);
    for (int i = 0; i < NIN; ++i) {
      c_stride[i] = KD.back().stride[i];
      r1_stride[i] = RD.back().stride[i];
      r0_stride[i] = rr2 ? RD[0].stride[i] : 0;
      mode[i] = c_stride[i] == 1 ? M_VEC : (c_stride[i] == 0 ? M_BCAST : M_GATHER);
      if (views[i].imm) mode[i] = M_IMM;
      if (views[i].iota) mode[i] = M_IOTA;
    }
    int vec = vec_width(mode);
    // Every thread keeps one accumulator per column of its vector: at most 64 bytes of them (int8 sums with their
    // int64 accumulators, 16384 x 16384: 2.2 TB/s with 8 columns per thread against 1.9 with 16; two long rows:
    // 0.51 against 0.28; int16 and float16 are indifferent, 4 columns per thread lose a quarter for int16)
    const int acc_cap = env_int("THX_RED_COL_ACCCAP", 64);
    while (vec > 1 && vec * r->acc_bytes > acc_cap) vec /= 2;
    auto vec_ok = [&](int v) {
      if (v == 1) return true;
      if (C % v) return false;
      if ((int64_t)cblock * v * r->acc_bytes > 32768) return false;
      for (int i = 0; i < NIN; ++i) {
        if (mode[i] != M_VEC) continue;
        if (((uintptr_t)views[i].ptr) % (size_t)(dtype_size(views[i].dtype) * v)) return false;
        if (r0_stride[i] % v || r1_stride[i] % v) return false;
        for (int d = 0; d < ko; ++d)
          if (KD[d].stride[i] % v) return false;
      }
      return true;
    };
    const int vec_full = vec;
    while (!vec_ok(vec)) vec /= 2;
    // Columns that are no whole number of vectors, or rows that start off a vector boundary ((100, 100, 13421)
    // float16 over the first two axes: 1.0 TB/s with 2-byte accesses): full-width vectors through element-aligned
    // pointers; the thread that owns the last, incomplete vector reads its columns one by one.
    int ua = 0;
    if (vec < vec_full && env_int("THX_RED_UA", 1)) {
      int v = vec_full;
      while (v > vec && ((int64_t)cblock * v * r->acc_bytes > 32768 || C < (int64_t)v * std::max(1, env_int("THX_RED_UA_MINVEC", 4)))) v /= 2;
      bool ok = v > vec;
      for (int i = 0; i < NIN; ++i)
        if (mode[i] == M_VEC && ((uintptr_t)views[i].ptr) % (size_t)dtype_size(views[i].dtype)) ok = false;
      if (ok) {
        vec = v;
        ua = 1;
      }
    }
    if ((int64_t)cblock * vec * r->acc_bytes > 65536)
      return fail(THX_ERR_UNSUPPORTED, "reduce: accumulator of %d bytes is too large for the column kernel", r->acc_bytes);
    const int64_t cvecs = ceil_div(C, (int64_t)vec);
    int tx = 1;
    // Up to seven rows: one row lane, 256 threads across, and every row of a thread's columns in flight at once
    // instead of four row lanes with one load each ((3, 22369621) float32 4.2 against 2.9 TB/s of input,
    // (7, 9586980) 5.0 against 4.5; from eight rows on the four lanes are the faster: 5.0 against 4.8)
    const bool one_lane = rows <= 7 && env_int("THX_RED_WIDE_TX", 1);
    const int tx_max = one_lane ? 256 : 64;
    while (tx < tx_max && tx < cvecs) tx *= 2;
    // Few column blocks for the device (a split into 4 or more row slices ahead): narrower and taller
    // blocks instead - 16 threads across (256-byte row segments for 4-byte elements), 512 threads,
    // 4 rows in flight per thread - leave 2 slices; measured 42.0 us against 47.1 us for the
    // (8192, 8192) float32 column sum.
    bool tall = false;
    if (!force_cb && tx == 64 && cvecs >= 64) {
      int64_t a0 = 1;
      for (int d = 0; d < ko; ++d) a0 *= KD[d].extent;
      if (a0 * ceil_div(cvecs, 64) * 4 <= target_col && (int64_t)512 * vec * r->acc_bytes <= 32768) {
        tall = true;
        cblock = 512;
        // rows that do not start on cache lines: a 256-byte segment touches three of them, a 1 KiB one nine
        // instead of eight ((67041, 1001) float32 5.4 against 4.3 TB/s, (100, 100, 6710) 4.5 against 3.7)
        tx = ua ? 64 : 16;
      }
    }
    const int force_tx = env_int("THX_RED_TX", 0);
    if (force_tx > 0) tx = force_tx;
    const int ty = cblock / tx;
    const int64_t cblocks = ceil_div(cvecs, tx);
    int64_t A = 1;
    for (int d = 0; d < ko; ++d) A *= KD[d].extent;
    const int64_t per_lane = ceil_div(rows, ty);
    int unr = per_lane >= 16 ? 8 : per_lane >= 4 ? 4 : per_lane >= 2 ? 2 : 1;
    if (one_lane && ty == 1) unr = rows <= 2 ? 2 : rows <= 4 ? 4 : 8;
    if (tall && unr > 4) unr = 4;
    if (tall && carries_positions && unr > 2) unr = 2;
    const int force_unr = env_int("THX_RED_UNR", 0);
    if (force_unr > 0) unr = force_unr;
    const int64_t blocks0 = A * cblocks;
    int64_t rps = rows;
    if (blocks0 * 2 <= target_col && rows >= (int64_t)ty * unr * 2) {
      int64_t want = std::min(ceil_div(target_col, blocks0), rows / ((int64_t)ty * unr));
      if (want > 1) {
        rps = round_up(ceil_div(rows, want), (int64_t)ty * unr);
        S = (int)ceil_div(rows, rps);
      }
    }
    const bool ticket = S > 1 && r->has_ticket && n_out <= THX_TICKET_WORDS && S < 65536 && env_int("THX_RED_TICKET", 1);
    one_launch = ticket;
    nblocks = blocks0 * S;
    gs = nblocks * cblock > max_dispatch;
    std::ostringstream key;
    key << "rc|k" << NK << (wide ? "|i64" : "|i32") << "|v" << vec << "|u" << unr << "|x" << tx << (cblock != 256 ? "|b" + std::to_string(cblock) : "") << "|r" << rr2 << (nt ? "|nt" + std::to_string(nt) : "") << (ticket ? "|tk" : "") << (gs ? "|gs" : "") << (ua ? "|ua" : "") << "|m";
    for (int i = 0; i < NIN; ++i) key << mode[i] << (i + 1 < NIN ? "," : "");
    plan = key.str() + (fast_div() ? "|fd" : "");
    auto it = r->plans.find(plan);
    if (it != r->plans.end() && (it->second.func || dry)) {
      k = it->second;
    } else if (fixed) {
      return not_loaded(r, plan);
    } else {
      const std::string entry = entry_name(r->name, plan);
      std::ostringstream s;
      s << device_prelude() << r->src
        << plan_struct(wide, {{"NK", NK}, {"VEC", vec}, {"UNR", unr}, {"BLOCK", cblock}, {"TX", tx}, {"RR2", rr2}, {"TICKET", ticket ? 1 : 0}, {"GS", gs ? 1 : 0}, {"UA", ua}}, mode, nt)
        << "extern \"C\" __global__ __launch_bounds__(" << cblock << ") void " << entry << "(thx::ColParams<" << r->name
        << "::NIN, " << r->name << "::NOUT, " << r->name << "::NEX, ThxPlan::NK, ThxPlan::IT> p) {\n  thx::red_col_body<" << r->name
        << ", ThxPlan>(p);\n}\n";
      rc = get_kernel(s.str(), entry, &k);
      if (rc) return rc;
      r->plans[plan] = k;
    }
    if (!dry && S > 1) {
      if (ticket) {
        partial = rt().ticket_words;
      } else {
        rc = partial_buffer(r, (size_t)S * n_out * r->acc_bytes, n_out, fixed, &partial);
        if (rc) return rc;
      }
    }
    for (int i = 0; i < NIN; ++i) pk.put<char*>(views[i].ptr);
    for (int i = 0; i < NIN; ++i) pk.put<uint64_t>(views[i].immval);
    for (int o = 0; o < NOUT; ++o) pk.put<char*>(outp[o]);
    for (uint64_t v : ex) pk.put<uint64_t>(v);
    for (int64_t v : exs) pk.put<int64_t>(v);
    pk.put<char*>(partial);
    pk.put<int64_t>(n_out);
    pk.put<int64_t>(nblocks);
    pk.put<int64_t>(rows);
    pk.put<int64_t>(rps);
    pk.put<int32_t>((int32_t)C);
    pk.put<int32_t>((int32_t)cblocks);
    pk.put<int32_t>(S);
    pk.put<int32_t>(0);
    for (int d = 0; d < NK; ++d) pk.put<FastDivH>(make_fastdiv(d < ko ? (uint64_t)KD[d].extent : 1));
    pk.put<FastDivH>(make_fastdiv((uint64_t)RD.back().extent));
    for (int i = 0; i < NIN; ++i)
      for (int d = 0; d < NK; ++d) pk.put_index(wide, d < ko ? KD[d].stride[i] : 0);
    for (int i = 0; i < NIN; ++i) pk.put_index(wide, r0_stride[i]);
    for (int i = 0; i < NIN; ++i) pk.put_index(wide, r1_stride[i]);
    for (int i = 0; i < NIN; ++i) pk.put_index(wide, c_stride[i]);
    pk.align(8);
    if (C >= (int64_t(1) << 31)) return fail(THX_ERR_UNSUPPORTED, "reduce: %lld kept columns", (long long)C);
    launch_block = cblock;
  } else if (form == STRIP) {
    const int64_t C = KD[0].extent, n = C * RD[0].extent;
    const int vec = strip_vec;
    const int64_t nvec = n / vec;
    std::vector<int> smode(NIN, M_VEC);
    int ua = 0;
    for (int i = 0; i < NIN; ++i) {
      if (views[i].imm) smode[i] = M_IMM;
      else if (((uintptr_t)views[i].ptr) % (size_t)(dtype_size(views[i].dtype) * vec)) ua = 1;
    }
    if (n >= (int64_t(1) << 31) - 65536) wide = true;
    const int64_t rounds = ceil_div(nvec, C * (int64_t)block);
    const int64_t G = std::max<int64_t>(1, std::min<int64_t>(rounds, (int64_t)cus * env_int("THX_RED_STRIP_BPC", 8)));
    S = (int)G;
    nblocks = G;
    std::ostringstream key;
    key << "rs|c" << C << (wide ? "|i64" : "|i32") << "|v" << vec << (nt ? "|nt" + std::to_string(nt) : "") << (ua ? "|ua" : "") << "|m";
    for (int i = 0; i < NIN; ++i) key << smode[i] << (i + 1 < NIN ? "," : "");
    plan = key.str() + (fast_div() ? "|fd" : "");
    auto it = r->plans.find(plan);
    if (it != r->plans.end() && (it->second.func || dry)) {
      k = it->second;
    } else if (fixed) {
      return not_loaded(r, plan);
    } else {
      const std::string entry = entry_name(r->name, plan);
      std::ostringstream s;
      s << device_prelude() << r->src
        << plan_struct(wide, {{"VEC", vec}, {"COLS", C}, {"BLOCK", block}, {"UA", ua}}, smode, nt)
        << "extern \"C\" __global__ __launch_bounds__(" << block << ") void " << entry << "(thx::StripParams<" << r->name
        << "::NIN, " << r->name << "::NOUT, " << r->name << "::NEX> p) {\n  thx::red_strip_body<" << r->name
        << ", ThxPlan>(p);\n}\n";
      rc = get_kernel(s.str(), entry, &k);
      if (rc) return rc;
      r->plans[plan] = k;
    }
    if (!dry && S > 1) {
      rc = partial_buffer(r, (size_t)S * n_out * r->acc_bytes, n_out, fixed, &partial);
      if (rc) return rc;
    }
    for (int i = 0; i < NIN; ++i) pk.put<char*>(views[i].ptr);
    for (int i = 0; i < NIN; ++i) pk.put<uint64_t>(views[i].immval);
    for (int o = 0; o < NOUT; ++o) pk.put<char*>(outp[o]);
    for (uint64_t v : ex) pk.put<uint64_t>(v);
    for (int64_t v : exs) pk.put<int64_t>(v);
    pk.put<char*>(partial);
    pk.put<int64_t>(nvec);
    pk.put<int64_t>(n);
    pk.put<int32_t>((int32_t)G);
    pk.put<int32_t>(0);
    pk.align(8);
  } else {
    const int NK = std::max(1, NKD);
    const int tpr = n_red >= 512 ? 256 : n_red >= 64 ? 64 : 1;
    std::vector<int> gmode(NIN, M_GATHER);
    nblocks = ceil_div(n_out, block / tpr);
    gs = nblocks * block > max_dispatch;
    std::ostringstream key;
    key << "rg|k" << NK << "|r" << NR << (wide ? "|i64" : "|i32") << "|t" << tpr << (gs ? "|gs" : "") << "|m";
    for (int i = 0; i < NIN; ++i) {
      if (views[i].imm) gmode[i] = M_IMM;
      if (views[i].iota) gmode[i] = M_IOTA;
      key << gmode[i] << (i + 1 < NIN ? "," : "");
    }
    plan = key.str() + (fast_div() ? "|fd" : "");
    auto it = r->plans.find(plan);
    if (it != r->plans.end() && (it->second.func || dry)) {
      k = it->second;
    } else if (fixed) {
      return not_loaded(r, plan);
    } else {
      const std::string entry = entry_name(r->name, plan);
      std::ostringstream s;
      s << device_prelude() << r->src
        << plan_struct(wide, {{"NK", NK}, {"NR", NR}, {"BLOCK", block}, {"TPR", tpr}, {"GS", gs ? 1 : 0}, {"UA", 0}}, gmode, 0)
        << "extern \"C\" __global__ __launch_bounds__(" << block << ") void " << entry << "(thx::GenParams<" << r->name
        << "::NIN, " << r->name << "::NOUT, " << r->name << "::NEX, ThxPlan::NK, ThxPlan::NR, ThxPlan::IT> p) {\n  thx::red_gen_body<" << r->name
        << ", ThxPlan>(p);\n}\n";
      rc = get_kernel(s.str(), entry, &k);
      if (rc) return rc;
      r->plans[plan] = k;
    }
    for (int i = 0; i < NIN; ++i) pk.put<char*>(views[i].ptr);
    for (int i = 0; i < NIN; ++i) pk.put<uint64_t>(views[i].immval);
    for (int o = 0; o < NOUT; ++o) pk.put<char*>(outp[o]);
    for (uint64_t v : ex) pk.put<uint64_t>(v);
    for (int64_t v : exs) pk.put<int64_t>(v);
    pk.put<int64_t>(n_out);
    pk.put<int64_t>(nblocks);
    pk.put<int64_t>(n_red);
    for (int d = 0; d < NK; ++d) pk.put<FastDivH>(make_fastdiv(d < NKD ? (uint64_t)KD[d].extent : 1));
    for (int d = 0; d < NR; ++d) pk.put<FastDivH>(make_fastdiv((uint64_t)RD[d].extent));
    for (int i = 0; i < NIN; ++i)
      for (int d = 0; d < NK; ++d) pk.put_index(wide, d < NKD ? KD[d].stride[i] : 0);
    for (int i = 0; i < NIN; ++i)
      for (int d = 0; d < NR; ++d) pk.put_index(wide, RD[d].stride[i]);
    pk.align(8);
  }

  set_last_plan(r->name + "|" + plan + (S > 1 ? "|s" + std::to_string(S) : ""));
  // One dispatch carries at most 2^32 - 1 work-items: beyond that the kernel is the striding variant (GS) and each
  // block takes several pieces of work.
  const int64_t grid = gs ? std::max<int64_t>(1, max_dispatch / launch_block) : nblocks;
  if (!dry) {
    rc = launch(k, r->name + "|" + plan, (unsigned)grid, launch_block, pk.buf.data(), pk.buf.size(), fixed);
    if (rc) return rc;
  }
  if (S > 1 && !one_launch)
    return reduce_final_pass(r, outp, ex, exs, partial, n_out, S, dry, fixed);
  return THX_OK;
}

extern "C" {

int thx_reduce_call(thx_reduce* r, const thx_array* ins, const uint8_t* reduce_mask, const thx_array* outs, int flags) {
  return reduce_impl(r, ins, reduce_mask, outs, flags, false);
}

int thx_reduce_call_static(thx_reduce* r, const thx_array* ins, const uint8_t* reduce_mask, const thx_array* outs,
                           int flags) {
  return reduce_impl(r, ins, reduce_mask, outs, flags, true);
}

}  // extern "C"
