// Row-chain planner: checks that every operand of an elementwise + row-reduction
// island can be walked row by row with unit column stride, picks the vector
// width and the number of threads per row, compiles on first use and launches.
#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <sstream>
#include <unordered_map>

#include "thx_internal.h"

struct thx_rowchain {
  std::string src, name;
  int n_in = 0, n_out = 0;
  std::vector<int32_t> dtypes, kinds;
  std::unordered_map<std::string, thx::Kernel> plans;
  std::unordered_map<std::string, int> spill_bytes;  // per plan: private memory per thread of the compiled kernel
  std::vector<int> axes;   // reduced axes of the full shape; empty: the last one
  bool has_held = false;   // the functor also carries the held form (`held`)
};

namespace thx {

enum { K_FULL = 0, K_ROW = 1, K_COL = 2, K_SCALAR = 3 };

// Stride between consecutive rows when the leading `nlead` dimensions collapse
// into one row index; false when they do not.
static bool row_stride(const int64_t* shape, const int64_t* stride, int nlead, int64_t* out) {
  int64_t st = 0;
  bool have = false;
  for (int d = nlead - 1; d >= 0; --d) {
    if (shape[d] == 1) continue;
    if (!have) {
      st = stride[d];
      have = true;
      *out = st;
      st *= shape[d];
    } else {
      if (stride[d] != st) return false;
      st *= shape[d];
    }
  }
  if (!have) *out = 0;
  return true;
}

static int env_int(const char* name, int dflt) {
  const char* v = getenv(name);
  return v ? atoi(v) : dflt;
}

// Stride (in elements) of dimensions [d0, d1) taken as one index, 0 when their extent is 1;
// false when they do not nest into a single stride.
static bool span_stride(const int64_t* shape, const int64_t* stride, int d0, int d1, int64_t* out) {
  int64_t st = 0;
  bool have = false;
  *out = 0;
  for (int d = d1 - 1; d >= d0; --d) {
    if (shape[d] == 1) continue;
    if (!have) {
      have = true;
      *out = stride[d];
      st = stride[d] * shape[d];
    } else {
      if (stride[d] != st) return false;
      st *= shape[d];
    }
  }
  return true;
}

}  // namespace thx

using namespace thx;

// The held form: one block per kept index keeps the whole reduce domain of that index (slabs of
// contiguous elements) on chip.  Reduced axes [0, k0) and (k1, nd) around the kept axes [k0, k1].
static int held_call(thx_rowchain* c, const thx_array* ins, const thx_array* outs, int flags) {
  const bool dry = (flags & THX_DRY_RUN) != 0;
  const int NIN = c->n_in, NOUT = c->n_out, NOPS = NIN + NOUT;
  if (!c->has_held) return fail(THX_ERR_UNSUPPORTED, "rowchain: this chain has no held form");
  if (env_int("THX_HELD", 1) == 0) return fail(THX_ERR_UNSUPPORTED, "rowchain: the held form is switched off");
  const thx_array* full = nullptr;
  for (int i = 0; i < NOPS && !full; ++i)
    if (c->kinds[i] == K_FULL) full = i < NIN ? &ins[i] : &outs[i - NIN];
  if (!full) return fail(THX_ERR_ARG, "rowchain: no full-shaped operand");
  const int nd = full->nd;
  if (nd < 1 || nd > THX_MAX_ND) return fail(THX_ERR_TYPE, "rowchain: rank %d", nd);
  std::vector<char> red(nd, 0);
  if (c->axes.empty()) {
    red[nd - 1] = 1;
  } else {
    for (int a : c->axes) {
      if (a < 0 || a >= nd) return fail(THX_ERR_ARG, "rowchain: reduced axis %d of a rank-%d operand", a, nd);
      red[a] = 1;
    }
  }
  int k0 = nd, k1 = -1;
  for (int d = 0; d < nd; ++d)
    if (!red[d]) {
      k0 = std::min(k0, d);
      k1 = std::max(k1, d);
    }
  if (k1 < 0) k0 = 0;   // nothing kept: one index, everything trails it
  for (int d = k0; d <= k1; ++d)
    if (red[d]) return fail(THX_ERR_UNSUPPORTED, "rowchain: kept axes are not adjacent");
  const int t0 = k1 + 1;   // trailing reduced axes [t0, nd), leading ones [0, k0)
  if (t0 >= nd) return fail(THX_ERR_UNSUPPORTED, "rowchain: no trailing reduced axis to walk with unit stride");
  int64_t A = 1, KX = 1, B = 1;
  for (int d = 0; d < k0; ++d) A *= full->shape[d];
  for (int d = k0; d <= k1; ++d) KX *= full->shape[d];
  for (int d = t0; d < nd; ++d) B *= full->shape[d];
  if (KX == 0) {
    set_last_plan("rh|empty");
    return THX_OK;
  }
  if (A == 0 || B == 0) return fail(THX_ERR_UNSUPPORTED, "rowchain: empty reduce domains are left to the unfused kernels (identity results)");

  std::vector<char*> ptr(NOPS, nullptr);
  std::vector<uint64_t> imm(NIN, 0);
  std::vector<int> is_imm(NIN, 0);
  std::vector<int64_t> sa(NOPS, 0), sk(NOPS, 0);   // in elements
  int maxsz = 1;
  for (int i = 0; i < NOPS; ++i) {
    const thx_array& a = i < NIN ? ins[i] : outs[i - NIN];
    const int kind = c->kinds[i];
    const int dt = a.dtype & ~(THX_HOST_SCALAR | THX_REUSED);
    if (dt != c->dtypes[i]) return fail(THX_ERR_TYPE, "rowchain: operand %d has dtype code %d, expected %d", i, dt, c->dtypes[i]);
    const int isz = dtype_size(dt);
    if (null_base(a, dry)) return fail(THX_ERR_ARG, "rowchain: operand %d has no base address", i);
    char* p = (char*)a.base + a.offset_bytes;
    if (a.dtype & THX_HOST_SCALAR) {
      if (kind != K_SCALAR || i >= NIN || isz > 8) return fail(THX_ERR_TYPE, "rowchain: operand %d cannot be a host scalar", i);
      memcpy(&imm[i], p, (size_t)isz);
      is_imm[i] = 1;
      continue;
    }
    if (((uintptr_t)p) % isz) return fail(THX_ERR_TYPE, "rowchain: operand %d is not aligned to its element size", i);
    ptr[i] = p;
    if (a.nd > THX_MAX_ND) return fail(THX_ERR_TYPE, "rowchain: operand %d has rank %d", i, a.nd);
    int64_t st[THX_MAX_ND];
    for (int d = 0; d < a.nd; ++d) {
      if (a.strides_bytes[d] % isz) return fail(THX_ERR_TYPE, "rowchain: operand %d has a stride that is not a multiple of its element size", i);
      st[d] = a.strides_bytes[d] / isz;
    }
    if (kind == K_FULL) {
      if (a.nd != nd) return fail(THX_ERR_TYPE, "rowchain: operand %d has rank %d, expected %d", i, a.nd, nd);
      for (int d = 0; d < nd; ++d)
        if (a.shape[d] != full->shape[d])
          return fail(THX_ERR_SHAPE, "Input dimension mis-match. (input[%d].shape[%d] = %lld, expected %lld)", i, d,
                      (long long)a.shape[d], (long long)full->shape[d]);
      int64_t sb = 0;
      if (!span_stride(a.shape, st, t0, nd, &sb) || (B > 1 && sb != 1))
        return fail(THX_ERR_UNSUPPORTED, "rowchain: operand %d is not contiguous along the trailing reduced axes", i);
      if (!span_stride(a.shape, st, 0, k0, &sa[i]) || !span_stride(a.shape, st, k0, k1 + 1, &sk[i]))
        return fail(THX_ERR_UNSUPPORTED, "rowchain: the leading or the kept dimensions of operand %d do not collapse", i);
      maxsz = std::max(maxsz, isz);
    } else if (kind == K_ROW) {
      // one value per kept index: rank nd with extent 1 on the reduced axes, or the kept axes alone
      const int nk = k1 >= k0 ? k1 - k0 + 1 : 0;
      if (a.nd == nd) {
        for (int d = 0; d < nd; ++d)
          if (a.shape[d] != (red[d] ? 1 : full->shape[d]))
            return fail(THX_ERR_SHAPE, "Input dimension mis-match. (input[%d].shape[%d] = %lld, expected %lld)", i, d,
                        (long long)a.shape[d], (long long)(red[d] ? 1 : full->shape[d]));
        if (!span_stride(a.shape, st, k0, k1 + 1, &sk[i]))
          return fail(THX_ERR_UNSUPPORTED, "rowchain: the kept dimensions of operand %d do not collapse", i);
      } else if (a.nd == nk) {
        for (int d = 0; d < nk; ++d)
          if (a.shape[d] != full->shape[k0 + d])
            return fail(THX_ERR_SHAPE, "Input dimension mis-match. (input[%d].shape[%d] = %lld, expected %lld)", i, d,
                        (long long)a.shape[d], (long long)full->shape[k0 + d]);
        if (!span_stride(a.shape, st, 0, nk, &sk[i]))
          return fail(THX_ERR_UNSUPPORTED, "rowchain: the dimensions of operand %d do not collapse", i);
      } else {
        return fail(THX_ERR_TYPE, "rowchain: per-index operand %d has rank %d", i, a.nd);
      }
    } else if (kind == K_COL) {
      return fail(THX_ERR_UNSUPPORTED, "rowchain: the held form takes no per-column operands");
    } else {
      for (int d = 0; d < a.nd; ++d)
        if (a.shape[d] != 1) return fail(THX_ERR_SHAPE, "rowchain: scalar operand %d has extent %lld", i, (long long)a.shape[d]);
    }
  }

  int vec = 16 / maxsz;
  auto vec_ok = [&](int v) {
    if (v == 1) return true;
    if (B % v) return false;
    for (int i = 0; i < NOPS; ++i) {
      if (c->kinds[i] != K_FULL) continue;
      const int isz = dtype_size(c->dtypes[i]);
      if (((uintptr_t)ptr[i]) % (size_t)(isz * v)) return false;
      if (sa[i] % v || sk[i] % v) return false;
    }
    return true;
  };
  while (!vec_ok(vec)) vec /= 2;
  const int64_t bv = B / vec;
  if (A * bv >= (int64_t(1) << 30)) return fail(THX_ERR_UNSUPPORTED, "rowchain: reduce domains of %lld elements", (long long)(A * B));
  const int64_t nvec = A * bv;
  // one wave for short domains (many kept indices of a few hundred elements: no barrier, no idle waves),
  // 256 threads up to 8 vectors each, 1024 beyond
  int block = nvec > 256 * 8 ? 1024 : nvec > 64 * 8 ? 256 : 64;
  {
    const int fb = env_int("THX_HELD_BLOCK", 0);
    if (fb == 64 || fb == 256 || fb == 512 || fb == 1024) block = fb;
  }
  const int nch = (int)((nvec + block - 1) / block);
  // what one thread holds: dwords per chunk and input; registers first, then LDS
  std::vector<int> words(NIN, 0), nlds(NIN, 0), ldsoff(NIN, 0);
  int total = 0;
  for (int i = 0; i < NIN; ++i)
    if (c->kinds[i] == K_FULL) {
      words[i] = (vec * dtype_size(c->dtypes[i]) + 3) / 4;
      total += nch * words[i];
    }
  const int reg_budget = env_int("THX_HELD_REGS", block == 1024 ? 64 : block == 512 ? 160 : 320);  // (64 / 256 threads: 512 registers a lane)
  const int lds_budget = 144 * 1024;
  int need = total - reg_budget, lds_bytes = 0;
  for (int i = 0; i < NIN && need > 0; ++i) {
    if (c->kinds[i] != K_FULL) continue;
    const int chunk_bytes = block * vec * dtype_size(c->dtypes[i]);
    ldsoff[i] = lds_bytes;
    while (need > 0 && nlds[i] < nch && lds_bytes + chunk_bytes <= lds_budget) {
      ++nlds[i];
      lds_bytes += chunk_bytes;
      need -= words[i];
    }
  }
  // (Streaming an operand that does not fit - reading it again in every loop through a ring of vectors in
  // flight - was measured on the batch-normalisation gradient, x held and g read twice: 92-100 us against
  // 84 us for the two separate kernels; one block per compute unit cannot overlap its arithmetic with its
  // own loads the way eight small blocks do.)
  if (need > 0)
    return fail(THX_ERR_UNSUPPORTED, "rowchain: reduce domains of %lld elements do not fit on chip (%d words per thread)",
                (long long)(A * B), total);
  int64_t moved = 0;
  for (int i = 0; i < NOPS; ++i)
    if (c->kinds[i] == K_FULL) moved += KX * A * B * dtype_size(c->dtypes[i]);
  // one block per kept index and compute unit: fewer indices than units leave the device idle, and the
  // kernels that split a reduce domain over many blocks do better
  const int64_t cus = rt().ready ? rt().cus : 256;
  if (env_int("THX_HELD", 1) != 2 && KX * 4 < cus * 3 && moved > (int64_t(16) << 20))
    return fail(THX_ERR_UNSUPPORTED, "rowchain: %lld kept indices leave most of %lld compute units idle", (long long)KX, (long long)cus);

  bool wide = false;
  for (int i = 0; i < NOPS; ++i) {
    const int isz = dtype_size(c->dtypes[i]);
    if (sa[i] < 0 || sk[i] < 0) wide = true;
    const int64_t span = ((A - 1) * sa[i] + (KX - 1) * sk[i] + B) * isz;
    if (span >= (int64_t(1) << 32) - 65536) wide = true;
  }
  // Never non-temporal by default: a block issues all its loads at once and its stores in one burst, and both
  // do better through the L2 (batch-normalisation gradient of a (256, 2048, 7, 7) float32 array, 616 MB moved:
  // 93.8 us against 132.6 us non-temporal; the forward pass of the float16 (256, 256, 28, 28) array 46 us
  // against 54 us)
  uint64_t nt_in = 0, nt_out = 0;
  if (nt_choice(0)) {
    for (int i = 0; i < NOPS && i < 64; ++i) {
      if (c->kinds[i] != K_FULL) continue;
      if (i < NIN) nt_in |= uint64_t(1) << i;
      else nt_out |= uint64_t(1) << (i - NIN);
    }
  }
  std::ostringstream key;
  const int nfull = (int)(nvec / block);
  key << "rh|v" << vec << "|n" << nch << (nfull != nch ? "p" : "") << "|b" << block << "|l";
  for (int i = 0; i < NIN; ++i) key << nlds[i] << (i + 1 < NIN ? "." : "");
  key << (wide ? "|i64" : "|i32");
  if (nt_in | nt_out) key << "|nt" << nt_in << "_" << nt_out;
  key << "|i";
  for (int i = 0; i < NIN; ++i) key << is_imm[i];
  const std::string plan = key.str() + (fast_div() ? "|fd" : "");
  set_last_plan(c->name + "|" + plan);
  Kernel k;
  auto it = c->plans.find(plan);
  if (it != c->plans.end() && (it->second.func || dry)) {
    k = it->second;
  } else {
    const std::string entry = entry_name(c->name, plan);
    std::ostringstream s;
    auto table = [&](const char* name, const std::vector<int>& v) {
      s << "  static constexpr int " << name << "(int i) {\n    constexpr int m[] = {";
      for (int i = 0; i < NIN; ++i) s << v[i] << (i + 1 < NIN ? ", " : "");
      s << "};\n    return m[i];\n  }\n";
    };
    s << device_prelude() << c->src << "\nstruct ThxPlan {\n  typedef " << (wide ? "long long" : "unsigned")
      << " IT;\n  enum { VEC = " << vec << ", NCH = " << nch << ", NFULL = " << nfull << ", BLOCK = " << block
      << ", LDS_BYTES = " << lds_bytes << " };\n  static constexpr unsigned long long NT = " << nt_in << "ull, NTO = " << nt_out << "ull;\n";
    table("imm", is_imm);
    table("nlds", nlds);
    table("ldsoff", ldsoff);
    s << "};\n"
      << "extern \"C\" __global__ __launch_bounds__(" << block << ") void " << entry << "(thx::HeldParams<" << c->name
      << "::NIN, " << c->name << "::NOUT, ThxPlan::IT> p) {\n  thx::heldchain_body<" << c->name << ", ThxPlan>(p);\n}\n";
    int rc = get_kernel(s.str(), entry, &k);
    if (rc) return rc;
    c->plans[plan] = k;
  }
  if (dry) return THX_OK;
  {
    // values that do not stay in registers go to private memory: more traffic than the kernels the caller falls back to
    auto sp = c->spill_bytes.find(plan);
    if (sp == c->spill_bytes.end()) {
      int bytes = 0;
      THX_HIP_CHECK(hipFuncGetAttribute(&bytes, HIP_FUNC_ATTRIBUTE_LOCAL_SIZE_BYTES, k.func));
      sp = c->spill_bytes.emplace(plan, bytes).first;
    }
    if (sp->second > 0 && env_int("THX_HELD", 1) != 2)
      return fail(THX_ERR_UNSUPPORTED, "rowchain: holding %lld elements per index needs %d bytes of private memory per thread",
                  (long long)(A * B), sp->second);
  }
  if (KX * block > 0xffffffffLL)
    return fail(THX_ERR_UNSUPPORTED, "rowchain: %lld blocks of %d exceed the work-items of one dispatch", (long long)KX, block);

  ParamPack pk;
  for (int i = 0; i < NIN; ++i) pk.put<char*>(ptr[i]);
  for (int i = 0; i < NIN; ++i) pk.put<uint64_t>(imm[i]);
  for (int i = 0; i < NOUT; ++i) pk.put<char*>(ptr[NIN + i]);
  auto put_bytes = [&](int64_t elems, int i) {
    const int64_t b = elems * dtype_size(c->dtypes[i]);
    if (wide) pk.put<int64_t>(b);
    else pk.put<uint32_t>((uint32_t)b);
  };
  for (int i = 0; i < NIN; ++i) put_bytes(sa[i], i);
  for (int i = 0; i < NIN; ++i) put_bytes(sk[i], i);
  for (int i = 0; i < NOUT; ++i) put_bytes(sa[NIN + i], NIN + i);
  for (int i = 0; i < NOUT; ++i) put_bytes(sk[NIN + i], NIN + i);
  pk.put<FastDivH>(make_fastdiv((uint64_t)bv));
  pk.put<uint32_t>((uint32_t)nvec);
  pk.put<uint32_t>((uint32_t)bv);
  pk.put<uint32_t>((uint32_t)(block / bv));
  pk.put<uint32_t>((uint32_t)(block % bv));
  pk.align(8);
  return launch(k, c->name + "|" + plan, (unsigned)KX, block, pk.buf.data(), pk.buf.size());
}

extern "C" {

int thx_rowchain_new(const char* functor_src, const char* functor_name, int n_in, int n_out, const int32_t* dtypes,
                     const int32_t* kinds, thx_rowchain** out) {
  if (!functor_src || !functor_name || !dtypes || !kinds || !out) return fail(THX_ERR_ARG, "thx_rowchain_new: null argument");
  if (n_in < 1 || n_out < 1) return fail(THX_ERR_ARG, "thx_rowchain_new: needs inputs and outputs");
  for (int i = 0; i < n_in + n_out; ++i) {
    if (!dtype_size(dtypes[i])) return fail(THX_ERR_TYPE, "thx_rowchain_new: unknown dtype code %d", dtypes[i]);
    if (kinds[i] < K_FULL || kinds[i] > K_SCALAR || (i >= n_in && kinds[i] > K_ROW))
      return fail(THX_ERR_ARG, "thx_rowchain_new: bad operand kind %d", kinds[i]);
  }
  thx_rowchain* c = new thx_rowchain;
  c->src = functor_src;
  c->name = functor_name;
  c->n_in = n_in;
  c->n_out = n_out;
  c->dtypes.assign(dtypes, dtypes + n_in + n_out);
  c->kinds.assign(kinds, kinds + n_in + n_out);
  c->has_held = c->src.find(" void held(") != std::string::npos;
  *out = c;
  return THX_OK;
}

int thx_rowchain_set_axes(thx_rowchain* c, int n_axes, const int32_t* axes) {
  if (!c || n_axes < 0 || (n_axes > 0 && !axes)) return fail(THX_ERR_ARG, "thx_rowchain_set_axes: bad argument");
  if (n_axes > THX_MAX_ND) return fail(THX_ERR_ARG, "thx_rowchain_set_axes: %d axes", n_axes);
  std::vector<int> v(axes, axes + n_axes);
  std::sort(v.begin(), v.end());
  for (size_t i = 0; i < v.size(); ++i)
    if (v[i] < 0 || v[i] >= THX_MAX_ND || (i && v[i] == v[i - 1])) return fail(THX_ERR_ARG, "thx_rowchain_set_axes: bad axis list");
  c->axes = v;
  return THX_OK;
}

int thx_rowchain_free(thx_rowchain* c) {
  delete c;
  return THX_OK;
}

int thx_rowchain_call(thx_rowchain* c, const thx_array* ins, const thx_array* outs, int flags) {
  if (!c || !ins || !outs) return fail(THX_ERR_ARG, "thx_rowchain_call: null argument");
  const bool dry = (flags & THX_DRY_RUN) != 0;
  if (!dry) {
    int rc = ensure_init();
    if (rc) return rc;
  }
  const int NIN = c->n_in, NOUT = c->n_out, NOPS = NIN + NOUT;
  // the full shape comes from the first full operand
  const thx_array* full = nullptr;
  for (int i = 0; i < NOPS && !full; ++i)
    if (c->kinds[i] == K_FULL) full = i < NIN ? &ins[i] : &outs[i - NIN];
  if (!full) return fail(THX_ERR_ARG, "rowchain: no full-shaped operand");
  const int nd = full->nd;
  if (nd < 1 || nd > THX_MAX_ND) return fail(THX_ERR_TYPE, "rowchain: rank %d", nd);
  if (!c->axes.empty() && !(c->axes.size() == 1 && c->axes[0] == nd - 1)) return held_call(c, ins, outs, flags);
  int64_t rows = 1;
  for (int d = 0; d < nd - 1; ++d) rows *= full->shape[d];
  const int64_t C = full->shape[nd - 1];
  if (rows == 0) {
    set_last_plan("rw|empty");
    return THX_OK;
  }
  if (C == 0) return fail(THX_ERR_UNSUPPORTED, "rowchain: empty rows are left to the unfused kernels (identity results)");
  if (C >= (int64_t(1) << 30)) return fail(THX_ERR_UNSUPPORTED, "rowchain: rows of %lld elements", (long long)C);

  std::vector<char*> ptr(NOPS, nullptr);
  std::vector<uint64_t> imm(NIN, 0);
  std::vector<int> is_imm(NIN, 0);
  std::vector<int64_t> rstride(NOPS, 0);
  int maxsz = 1;
  for (int i = 0; i < NOPS; ++i) {
    const thx_array& a = i < NIN ? ins[i] : outs[i - NIN];
    const int kind = c->kinds[i];
    const int dt = a.dtype & ~(THX_HOST_SCALAR | THX_REUSED);
    if (dt != c->dtypes[i]) return fail(THX_ERR_TYPE, "rowchain: operand %d has dtype code %d, expected %d", i, dt, c->dtypes[i]);
    const int isz = dtype_size(dt);
    if (null_base(a, dry)) return fail(THX_ERR_ARG, "rowchain: operand %d has no base address", i);
    char* p = (char*)a.base + a.offset_bytes;
    if (a.dtype & THX_HOST_SCALAR) {
      if (kind != K_SCALAR || i >= NIN || isz > 8) return fail(THX_ERR_TYPE, "rowchain: operand %d cannot be a host scalar", i);
      memcpy(&imm[i], p, (size_t)isz);
      is_imm[i] = 1;
      continue;
    }
    if (((uintptr_t)p) % isz) return fail(THX_ERR_TYPE, "rowchain: operand %d is not aligned to its element size", i);
    ptr[i] = p;
    int64_t st[THX_MAX_ND];
    for (int d = 0; d < a.nd; ++d) {
      if (a.strides_bytes[d] % isz) return fail(THX_ERR_TYPE, "rowchain: operand %d has a stride that is not a multiple of its element size", i);
      st[d] = a.strides_bytes[d] / isz;
    }
    if (kind == K_FULL) {
      if (a.nd != nd) return fail(THX_ERR_TYPE, "rowchain: operand %d has rank %d, expected %d", i, a.nd, nd);
      for (int d = 0; d < nd; ++d)
        if (a.shape[d] != full->shape[d])
          return fail(THX_ERR_SHAPE, "Input dimension mis-match. (input[%d].shape[%d] = %lld, expected %lld)", i, d,
                      (long long)a.shape[d], (long long)full->shape[d]);
      if (C > 1 && st[nd - 1] != 1) return fail(THX_ERR_UNSUPPORTED, "rowchain: operand %d is not contiguous along its rows", i);
      if (!row_stride(a.shape, st, nd - 1, &rstride[i]))
        return fail(THX_ERR_UNSUPPORTED, "rowchain: the leading dimensions of operand %d do not collapse", i);
      maxsz = std::max(maxsz, isz);
    } else if (kind == K_ROW) {
      // rank nd with a trailing extent of 1, or rank nd - 1
      if (a.nd != nd && a.nd != nd - 1) return fail(THX_ERR_TYPE, "rowchain: per-row operand %d has rank %d", i, a.nd);
      if (a.nd == nd && a.shape[nd - 1] != 1) return fail(THX_ERR_SHAPE, "rowchain: per-row operand %d has %lld columns", i, (long long)a.shape[nd - 1]);
      for (int d = 0; d < nd - 1; ++d)
        if (a.shape[d] != full->shape[d])
          return fail(THX_ERR_SHAPE, "Input dimension mis-match. (input[%d].shape[%d] = %lld, expected %lld)", i, d,
                      (long long)a.shape[d], (long long)full->shape[d]);
      if (!row_stride(a.shape, st, nd - 1, &rstride[i]))
        return fail(THX_ERR_UNSUPPORTED, "rowchain: the leading dimensions of operand %d do not collapse", i);
    } else if (kind == K_COL) {
      if (a.nd != nd || a.shape[nd - 1] != C) return fail(THX_ERR_SHAPE, "rowchain: per-column operand %d has the wrong shape", i);
      for (int d = 0; d < nd - 1; ++d)
        if (a.shape[d] != 1) return fail(THX_ERR_SHAPE, "rowchain: per-column operand %d has leading extent %lld", i, (long long)a.shape[d]);
      if (C > 1 && st[nd - 1] != 1) return fail(THX_ERR_UNSUPPORTED, "rowchain: operand %d is not contiguous", i);
      rstride[i] = 0;
      maxsz = std::max(maxsz, isz);
    } else {
      for (int d = 0; d < a.nd; ++d)
        if (a.shape[d] != 1) return fail(THX_ERR_SHAPE, "rowchain: scalar operand %d has extent %lld", i, (long long)a.shape[d]);
    }
  }

  int vec = 16 / maxsz;
  auto vec_ok = [&](int v) {
    if (v == 1) return true;
    if (C % v) return false;
    for (int i = 0; i < NOPS; ++i) {
      if (c->kinds[i] != K_FULL && c->kinds[i] != K_COL) continue;
      const int isz = dtype_size(c->dtypes[i]);
      if (((uintptr_t)ptr[i]) % (size_t)(isz * v)) return false;
      if (rstride[i] % v) return false;
    }
    return true;
  };
  const int vec_full = vec;
  while (!vec_ok(vec)) vec /= 2;
  // Rows of 1001 or 50257 elements, or rows that start off a vector boundary: full-width vectors through
  // element-aligned pointers, the last one of a row moved back to end with the row (a (33520, 1001) float32 softmax:
  // 51.3 us with 4-byte accesses against 41.2 us for 1000 columns; float16: 117 against 66 us)
  int ua = 0;
  if (vec < vec_full && !(getenv("THX_ROW_UA") && atoi(getenv("THX_ROW_UA")) == 0)) {
    bool ok = true;
    for (int i = 0; i < NOPS; ++i)
      if ((c->kinds[i] == K_FULL || c->kinds[i] == K_COL) && ((uintptr_t)ptr[i]) % (size_t)dtype_size(c->dtypes[i])) ok = false;
    int v = vec_full;
    while (v > vec && C < (int64_t)v * 2) v /= 2;
    if (ok && v > vec) {
      vec = v;
      ua = 1;
    }
  }
  const int64_t cv = (C + vec - 1) / vec;
  int tpr, nch;
  if (cv <= 8 * 64) {
    tpr = 64;
    nch = (int)((cv + 63) / 64);
  } else if (cv <= 16 * 256) {
    tpr = 256;
    nch = (int)((cv + 255) / 256);
  } else if (cv <= 16 * 1024 && !(getenv("THX_ROW_BIG") && atoi(getenv("THX_ROW_BIG")) == 0)) {
    // one block of 1024 threads per row (128 registers per thread: chains that keep several row-sized
    // values alive spill, and are turned away below)
    tpr = 1024;
    nch = (int)((cv + 1023) / 1024);
  } else {
    // longer rows stay on chip in their storage type if the chain has the held form
    if (c->has_held) return held_call(c, ins, outs, flags);
    return fail(THX_ERR_UNSUPPORTED, "rowchain: rows of %lld elements do not fit in registers", (long long)C);
  }
  const int force_tpr = getenv("THX_ROW_TPR") ? atoi(getenv("THX_ROW_TPR")) : 0;
  if (force_tpr == 256 || force_tpr == 64) {
    tpr = force_tpr;
    nch = (int)((cv + tpr - 1) / tpr);
    if (nch > 32) return fail(THX_ERR_UNSUPPORTED, "rowchain: forced threads per row give %d chunks", nch);
  }
  bool wide = false;
  for (int i = 0; i < NOPS; ++i) {
    int64_t span = (rows - 1) * (rstride[i] < 0 ? -rstride[i] : rstride[i]) + C;
    if (span >= (int64_t(1) << 31) - 65536) wide = true;
  }
  const int block = tpr == 1024 ? 1024 : 256;
  int64_t moved = 0;
  for (int i = 0; i < NOPS; ++i)
    if (c->kinds[i] == K_FULL) moved += rows * C * dtype_size(c->dtypes[i]);
  // non-temporal per operand: the call-wide choice, withdrawn from operands a later call reads
  uint64_t nt_in = 0, nt_out = 0;
  if (nt_streaming(moved)) {
    const bool forced = getenv("THX_NT") != nullptr;
    for (int i = 0; i < NOPS && i < 64; ++i) {
      const thx_array& a = i < NIN ? ins[i] : outs[i - NIN];
      if (!forced && (a.dtype & THX_REUSED)) continue;
      if (i < NIN) nt_in |= uint64_t(1) << i;
      else nt_out |= uint64_t(1) << (i - NIN);
    }
  }

  std::ostringstream key;
  key << "rw|v" << vec << "|n" << nch << "|t" << tpr << (wide ? "|i64" : "|i32") << (ua ? "|ua" : "");
  if (nt_in | nt_out) key << "|nt" << nt_in << "_" << nt_out;
  key << "|i";
  for (int i = 0; i < NIN; ++i) key << is_imm[i];
  const std::string plan = key.str() + (fast_div() ? "|fd" : "");
  set_last_plan(c->name + "|" + plan);
  Kernel k;
  auto it = c->plans.find(plan);
  if (it != c->plans.end() && (it->second.func || dry)) {
    k = it->second;
  } else {
    const std::string entry = entry_name(c->name, plan);
    std::ostringstream s;
    s << device_prelude() << c->src << "\nstruct ThxPlan {\n  typedef " << (wide ? "long long" : "int")
      << " IT;\n  enum { VEC = " << vec << ", NCH = " << nch << ", TPR = " << tpr << ", BLOCK = " << block
      << ", UA = " << ua << " };\n  static constexpr unsigned long long NT = " << nt_in << "ull, NTO = " << nt_out
      << "ull;\n  static constexpr int imm(int i) {\n    constexpr int m[] = {";
    for (int i = 0; i < NIN; ++i) s << is_imm[i] << (i + 1 < NIN ? ", " : "");
    s << "};\n    return m[i];\n  }\n};\n"
      << "extern \"C\" __global__ __launch_bounds__(" << block << ") void " << entry << "(thx::RowChainParams<" << c->name
      << "::NIN, " << c->name << "::NOUT, ThxPlan::IT> p) {\n  thx::rowchain_body<" << c->name << ", ThxPlan>(p);\n}\n";
    int rc = get_kernel(s.str(), entry, &k);
    if (rc) return rc;
    c->plans[plan] = k;
  }
  if (dry) return THX_OK;
  if (tpr == 1024) {
    // a row per 1024-thread block leaves 128 registers a thread; a chain that needs more keeps its rows
    // in private memory, which costs more traffic than the separate kernels the caller falls back to
    auto sp = c->spill_bytes.find(plan);
    if (sp == c->spill_bytes.end()) {
      int bytes = 0;
      THX_HIP_CHECK(hipFuncGetAttribute(&bytes, HIP_FUNC_ATTRIBUTE_LOCAL_SIZE_BYTES, k.func));
      sp = c->spill_bytes.emplace(plan, bytes).first;
    }
    if (sp->second > 0 && !(getenv("THX_ROW_BIG") && atoi(getenv("THX_ROW_BIG")) == 2)) {
      if (c->has_held) return held_call(c, ins, outs, flags);
      return fail(THX_ERR_UNSUPPORTED, "rowchain: rows of %lld elements need %d bytes of private memory per thread",
                  (long long)C, sp->second);
    }
  }

  ParamPack pk;
  for (int i = 0; i < NIN; ++i) pk.put<char*>(ptr[i]);
  for (int i = 0; i < NIN; ++i) pk.put<uint64_t>(imm[i]);
  for (int i = 0; i < NOUT; ++i) pk.put<char*>(ptr[NIN + i]);
  pk.put<int64_t>(rows);
  pk.put<int32_t>((int32_t)C);
  pk.put<int32_t>((int32_t)cv);
  for (int i = 0; i < NIN; ++i) pk.put_index(wide, rstride[i]);
  for (int i = 0; i < NOUT; ++i) pk.put_index(wide, rstride[NIN + i]);
  pk.align(8);
  const int rpb = block / tpr;
  const int64_t grid = (rows + rpb - 1) / rpb;
  if (grid * block > 0xffffffffLL)
    return fail(THX_ERR_UNSUPPORTED, "rowchain: %lld blocks of %d exceed the work-items of one dispatch", (long long)grid, block);
  return launch(k, c->name + "|" + plan, (unsigned)grid, block, pk.buf.data(), pk.buf.size());
}

}  // extern "C"
