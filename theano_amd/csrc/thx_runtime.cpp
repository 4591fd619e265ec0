// Runtime of libthx_hip.so: device set-up, pooled memory, transfers, the hipRTC
// compile path with its two caches, launches and event timing.
#include <hip/hip_runtime.h>
#include <hip/hiprtc.h>
#include <sys/stat.h>
#include <unistd.h>

#include <cctype>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <mutex>
#include <sstream>
#include <unordered_map>

#include "thx_internal.h"

// Fixed scratch memory for thx_reduce_call_static: partial results of a split reduction, laid out
// [slice][output] like the allocated scratch buffer.  It is part of the library's code object, so
// every GPU the library runs on holds its own copy from load time until the process ends, and no
// call ever has to allocate it.  In host code the name `scratch` is only a handle for
// hipGetSymbolAddress: the device address is resolved once per device in thx_init and that
// address is what kernels and copies receive.  (No `used` attribute here: it makes the compiler emit
// the variable before it has seen the host code that refers to it, the device symbol then stays
// local, and the runtime, which finds the array by name, aborts in hipGetSymbolAddress.)
static __device__ __align__(256) unsigned char scratch[THX_STATIC_SCRATCH_BYTES];

// One 64-bit word per result for reductions that finish through a single atomic add per slice
// (kernels/thx_reduce.h, ticket_finish).  Zero when the library is loaded; every kernel that uses
// the words leaves them zero.  Resolved like `scratch`.
static __device__ __align__(256) unsigned long long ticket_words[THX_TICKET_WORDS];

namespace thx {

// ---------------------------------------------------------------------------
// errors
static thread_local std::string g_error;
static thread_local std::string g_plan;

int fail(int code, const char* fmt, ...) {
  char buf[4096];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof buf, fmt, ap);
  va_end(ap);
  g_error = buf;
  return code;
}
void set_last_plan(const std::string& plan) { g_plan = plan; }

// ---------------------------------------------------------------------------
// state
static std::mutex g_mu;
Runtime& rt() {
  static Runtime r;
  return r;
}

static std::string g_cache_dir;
static bool g_cache_dir_set = false;
static int64_t g_n_compiled = 0, g_n_disk = 0, g_n_mem = 0;
static std::unordered_map<std::string, Kernel> g_kernels;  // by hash of source

// pool
static std::unordered_map<size_t, std::vector<void*>> g_free;
static std::unordered_map<void*, size_t> g_live;

enum { kMaxDevices = 64 };
static char* g_static_scratch[kMaxDevices] = {nullptr};  // device address of `scratch`, per device
static char* g_ticket_words[kMaxDevices] = {nullptr};    // device address of `ticket_words`, per device

// profiling
struct ProfRec {
  std::string plan;
  hipEvent_t a, b;
};
static bool g_profiling = false;
static std::vector<ProfRec> g_prof;
static hipEvent_t g_t0 = nullptr, g_t1 = nullptr;

static int init_locked(int device) {
  Runtime& r = rt();
  if (r.ready) {
    if (device >= 0 && device != r.device)
      return fail(THX_ERR_ARG, "thx_init: already bound to device %d, asked for %d", r.device, device);
    return THX_OK;
  }
  if (device < 0) device = 0;
  int count = 0;
  hipError_t e = hipGetDeviceCount(&count);
  if (e != hipSuccess || count == 0)
    return fail(THX_ERR_HIP, "thx_init: no HIP device is visible (%s)", hipGetErrorString(e));
  if (device >= count || device >= kMaxDevices) return fail(THX_ERR_ARG, "thx_init: device %d of %d", device, count);
  THX_HIP_CHECK(hipSetDevice(device));
  if (!g_static_scratch[device]) {  // with `device` current: each GPU has the array at its own address
    void* p = nullptr;
    hipError_t se = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (se != hipSuccess || !p)
      return fail(THX_ERR_HIP, "thx_init: hipGetSymbolAddress(scratch) failed on device %d: %s", device,
                  hipGetErrorString(se));
    g_static_scratch[device] = (char*)p;
  }
  r.static_scratch = g_static_scratch[device];
  if (!g_ticket_words[device]) {
    void* p = nullptr;
    hipError_t se = hipGetSymbolAddress(&p, HIP_SYMBOL(ticket_words));
    if (se != hipSuccess || !p)
      return fail(THX_ERR_HIP, "thx_init: hipGetSymbolAddress(ticket_words) failed on device %d: %s", device,
                  hipGetErrorString(se));
    g_ticket_words[device] = (char*)p;
  }
  r.ticket_words = g_ticket_words[device];
  hipDeviceProp_t prop;
  THX_HIP_CHECK(hipGetDeviceProperties(&prop, device));
  r.device = device;
  r.cus = prop.multiProcessorCount;
  r.hbm = (int64_t)prop.totalGlobalMem;
  r.arch = prop.gcnArchName;
  r.arch_base = r.arch.substr(0, r.arch.find(':'));
  THX_HIP_CHECK(hipStreamCreateWithFlags(&r.stream, hipStreamNonBlocking));
  THX_HIP_CHECK(hipEventCreate(&g_t0));
  THX_HIP_CHECK(hipEventCreate(&g_t1));
  r.ready = true;
  return THX_OK;
}

int ensure_init() {
  std::lock_guard<std::mutex> lk(g_mu);
  return init_locked(-1);
}

// Recorded launch sequences keep the scratch address they were recorded with: while any of them is alive
// a scratch buffer that has become too small is set aside, not freed, and released with the last graph.
static bool g_capturing = false;
static int g_live_graphs = 0;
static std::vector<void*> g_retired_scratch;

static void release_retired_scratch() {
  for (void* p : g_retired_scratch) (void)hipFree(p);
  g_retired_scratch.clear();
}

int ensure_scratch(size_t bytes) {
  Runtime& r = rt();
  if (bytes <= r.scratch_bytes) return THX_OK;
  if (g_capturing)
    return fail(THX_ERR_ARG,
                "a recording needs %zu bytes of reduction scratch, %zu are allocated: run the same calls once before "
                "recording them (growing the buffer waits for the device, which ends a recording)",
                bytes, r.scratch_bytes);
  if (r.scratch) {
    if (g_live_graphs > 0) {
      g_retired_scratch.push_back(r.scratch);
    } else {
      THX_HIP_CHECK(hipStreamSynchronize(r.stream));
      THX_HIP_CHECK(hipFree(r.scratch));
    }
    r.scratch = nullptr;
    r.scratch_bytes = 0;
  }
  size_t want = bytes < (size_t(8) << 20) ? (size_t(8) << 20) : bytes;
  void* p = nullptr;
  if (hipMalloc(&p, want) != hipSuccess)
    return fail(THX_ERR_MEMORY, "cannot allocate %zu bytes of reduction scratch", want);
  r.scratch = (char*)p;
  r.scratch_bytes = want;
  return THX_OK;
}

// ---------------------------------------------------------------------------
// helpers
int dtype_size(int dtype) {
  static const int sz[THX_NDTYPES] = {1, 1, 1, 2, 2, 4, 4, 8, 8, 2, 4, 8, 8, 16};
  return (dtype >= 0 && dtype < THX_NDTYPES) ? sz[dtype] : 0;
}
const char* dtype_ctype(int dtype) {
  static const char* nm[THX_NDTYPES] = {"thx_bool", "thx_i8",  "thx_u8",  "thx_i16", "thx_u16", "thx_i32",
                                        "thx_u32",  "thx_i64", "thx_u64", "thx_f16", "thx_f32", "thx_f64",
                                        "thx_c64",  "thx_c128"};
  return (dtype >= 0 && dtype < THX_NDTYPES) ? nm[dtype] : "void";
}

FastDivH make_fastdiv(uint64_t d) {
  FastDivH f{0, 0, (uint32_t)d, 0};
  if (d < 2 || d >= (uint64_t(1) << 31)) return f;  // 64-bit plans divide directly; d = 1 slots are never divided by
  unsigned L = 0;
  while ((uint64_t(1) << L) < d) ++L;
  const unsigned __int128 one = 1;
  const unsigned __int128 num = one << (31 + L);
  f.m = (uint32_t)((num + d - 1) / d);
  f.s = L - 1;
  return f;
}

int gather_inputs(const char* what, const thx_array* ins, int n_in, const int32_t* dtypes, int flags, int* nd_out,
                  int64_t* shape, std::vector<View>* views) {
  if (n_in < 1) return fail(THX_ERR_ARG, "%s: needs at least one input", what);
  const int nd = ins[0].nd;
  if (nd < 0 || nd > THX_MAX_ND) return fail(THX_ERR_TYPE, "%s: rank %d is outside 0..%d", what, nd, THX_MAX_ND);
  for (int d = 0; d < nd; ++d) shape[d] = 1;
  int owner[THX_MAX_ND];
  for (int d = 0; d < nd; ++d) owner[d] = -1;
  for (int i = 0; i < n_in; ++i) {
    if (ins[i].nd != nd)
      return fail(THX_ERR_TYPE, "%s: input %d has rank %d, expected %d", what, i, ins[i].nd, nd);
    if ((ins[i].dtype & ~(THX_HOST_SCALAR | THX_INDEX | THX_REUSED)) != dtypes[i])
      return fail(THX_ERR_TYPE, "%s: input %d has dtype code %d, the operation was built for %d", what, i,
                  ins[i].dtype & ~(THX_HOST_SCALAR | THX_INDEX | THX_REUSED), dtypes[i]);
    for (int d = 0; d < nd; ++d) {
      const int64_t s = ins[i].shape[d];
      if (s < 0) return fail(THX_ERR_ARG, "%s: negative extent", what);
      if (owner[d] < 0) {
        shape[d] = s;
        owner[d] = i;
      } else if (s != shape[d]) {
        const bool can = (flags & THX_BROADCAST) != 0;
        if (can && shape[d] == 1) {
          shape[d] = s;
          owner[d] = i;
        } else if (!(can && s == 1)) {
          return fail(THX_ERR_SHAPE,
                      "Input dimension mis-match. (input[%d].shape[%d] = %lld, input[%d].shape[%d] = %lld)",
                      owner[d], d, (long long)shape[d], i, d, (long long)s);
        }
      }
    }
  }
  views->assign(n_in, View());
  for (int i = 0; i < n_in; ++i) {
    View& v = (*views)[i];
    if (null_base(ins[i], (flags & THX_DRY_RUN) != 0)) return fail(THX_ERR_ARG, "%s: input %d has no base address", what, i);
    v.ptr = (char*)ins[i].base + ins[i].offset_bytes;
    v.reused = (ins[i].dtype & THX_REUSED) != 0;
    v.dtype = ins[i].dtype & ~(THX_HOST_SCALAR | THX_INDEX | THX_REUSED);
    const int isz = dtype_size(v.dtype);
    if (!isz) return fail(THX_ERR_TYPE, "%s: unknown dtype code %d", what, v.dtype);
    if (ins[i].dtype & THX_INDEX) {  // no memory behind it; the caller that supports it fills in the multipliers
      if (v.dtype != THX_I64) return fail(THX_ERR_TYPE, "%s: index operand %d must be int64", what, i);
      for (int d = 0; d < nd; ++d)
        if (ins[i].shape[d] != 1) return fail(THX_ERR_TYPE, "%s: index operand %d must have extent 1 everywhere", what, i);
      v.ptr = nullptr;
      v.iota = true;
      continue;
    }
    if (ins[i].dtype & THX_HOST_SCALAR) {
      for (int d = 0; d < nd; ++d)
        if (ins[i].shape[d] != 1) return fail(THX_ERR_TYPE, "%s: host scalar input %d must have extent 1 everywhere", what, i);
      if (!v.ptr) return fail(THX_ERR_ARG, "%s: host scalar input %d is null", what, i);
      if (isz > 8) return fail(THX_ERR_TYPE, "%s: host scalar input %d: values of %d bytes do not travel by value", what, i, isz);
      v.imm = true;
      memcpy(&v.immval, v.ptr, (size_t)isz);
      v.ptr = nullptr;
      continue;
    }
    if (((uintptr_t)v.ptr) % isz)
      return fail(THX_ERR_TYPE, "%s: input %d is not aligned to its element size", what, i);
    for (int d = 0; d < nd; ++d) {
      if (ins[i].shape[d] == 1 && shape[d] != 1) {
        v.stride[d] = 0;
      } else {
        if (ins[i].strides_bytes[d] % isz)
          return fail(THX_ERR_TYPE, "%s: input %d stride %lld is not a multiple of its element size", what, i,
                      (long long)ins[i].strides_bytes[d]);
        v.stride[d] = ins[i].strides_bytes[d] / isz;
      }
    }
  }
  *nd_out = nd;
  return THX_OK;
}

// ---------------------------------------------------------------------------
// hipRTC
bool fast_div() {
  const char* env = getenv("THX_FAST_DIV");
  return env ? atoi(env) != 0 : true;
}

int nt_choice(int family_default) {
  const char* env = getenv("THX_NT");
  return env ? (atoi(env) != 0) : family_default;
}

uint64_t nt_mask(int nt, const std::vector<View>& views) {
  if (!nt) return 0;
  const bool forced = getenv("THX_NT") != nullptr;
  uint64_t m = 0;
  for (size_t i = 0; i < views.size() && i < 64; ++i)
    if (forced || !views[i].reused) m |= uint64_t(1) << i;
  return m;
}

int nt_streaming(int64_t moved) { return nt_choice(moved >= (int64_t(288) << 20)); }

static uint64_t fnv1a(const std::string& s, uint64_t h) {
  for (unsigned char c : s) {
    h ^= c;
    h *= 1099511628211ULL;
  }
  return h;
}

// $THX_FP_CONTRACT = on | off | fast: how the compiler may fuse a multiply with a following add.  Unset, the
// compiler's default for device code (fast: across statements) stays.
static const char* fp_contract() {
  const char* v = getenv("THX_FP_CONTRACT");
  if (!v) return "";
  return !strcmp(v, "on") ? "on" : !strcmp(v, "off") ? "off" : !strcmp(v, "fast") ? "fast" : "";
}

static std::string source_hash(const std::string& src, const std::string& arch) {
  int maj = 0, min = 0;
  hiprtcVersion(&maj, &min);
  std::string salted = src + "\n//" + arch + "/" + std::to_string(maj) + "." + std::to_string(min) +
                       (fast_div() ? "/fd" : "") + (fp_contract()[0] ? std::string("/c") + fp_contract() : std::string());
  char buf[40];
  snprintf(buf, sizeof buf, "%016llx%016llx", (unsigned long long)fnv1a(salted, 1469598103934665603ULL),
           (unsigned long long)fnv1a(salted, 0x9e3779b97f4a7c15ULL));
  return buf;
}

static const std::string& cache_dir() {
  if (!g_cache_dir_set) {
    const char* env = getenv("THX_CACHE_DIR");
    if (env) {
      g_cache_dir = env;
    } else {
      const char* home = getenv("HOME");
      g_cache_dir = std::string(home ? home : "/tmp") + "/.cache/thx_hip";
    }
    g_cache_dir_set = true;
  }
  return g_cache_dir;
}

static void mkdirs(const std::string& path) {
  std::string cur;
  for (size_t i = 0; i <= path.size(); ++i) {
    if (i == path.size() || path[i] == '/') {
      if (!cur.empty()) mkdir(cur.c_str(), 0777);
    }
    if (i < path.size()) cur += path[i];
  }
}

static std::string target_arch() {
  if (rt().ready) return rt().arch_base;
  const char* env = getenv("THX_ARCH");
  return env ? env : "gfx950";
}

static int compile_source(const std::string& src, const std::string& arch, std::vector<char>* code) {
  hiprtcProgram prog;
  hiprtcResult r = hiprtcCreateProgram(&prog, src.c_str(), "thx_kernel.hip", 0, nullptr, nullptr);
  if (r != HIPRTC_SUCCESS) return fail(THX_ERR_HIP, "hiprtcCreateProgram: %s", hiprtcGetErrorString(r));
  const std::string archopt = "--offload-arch=" + arch;
  // Packed FP32 instructions are disabled for every kernel of this library.
  std::vector<const char*> opts = {archopt.c_str(), "-O3", "-std=c++17", "-Xclang", "-target-feature", "-Xclang",
                                   "-packed-fp32-ops"};
  // float32 division and sqrt within 2.5 ulp instead of correctly rounded: a tenth of the instructions,
  // and two orders of magnitude inside the float32 parity tolerance (rtol 1e-5)
  if (fast_div()) {
    opts.push_back("-fno-hip-fp32-correctly-rounded-divide-sqrt");
    opts.push_back("-DTHX_FAST_DIV");
  }
  const std::string contract = std::string("-ffp-contract=") + fp_contract();
  if (fp_contract()[0]) opts.push_back(contract.c_str());
  r = hiprtcCompileProgram(prog, (int)opts.size(), opts.data());
  if (r != HIPRTC_SUCCESS) {
    size_t n = 0;
    hiprtcGetProgramLogSize(prog, &n);
    std::string log(n, '\0');
    if (n) hiprtcGetProgramLog(prog, &log[0]);
    hiprtcDestroyProgram(&prog);
    if (log.size() > 3500) log.resize(3500);
    return fail(THX_ERR_COMPILE, "hipRTC compilation failed (%s):\n%s", hiprtcGetErrorString(r), log.c_str());
  }
  size_t n = 0;
  hiprtcGetCodeSize(prog, &n);
  code->resize(n);
  hiprtcGetCode(prog, code->data());
  hiprtcDestroyProgram(&prog);
  return THX_OK;
}

// Is `b` a whole 64-bit ELF file?  The module loader does not check what it is given - half a code object or
// a file of something else ends the process inside it - so a cached file is loaded only if its header, its
// program and section header tables and every section's bytes lie inside the file (the section header table is
// the last thing in a code object: a file that was cut short fails here).
static bool elf_complete(const std::vector<char>& b) {
  const size_t n = b.size();
  if (n < 64 || memcmp(b.data(), "\177ELF", 4) != 0 || b[4] != 2 /* ELFCLASS64 */ || b[5] != 1 /* little-endian */) return false;
  auto u16 = [&](size_t off) { uint16_t v; memcpy(&v, b.data() + off, 2); return (uint64_t)v; };
  auto u32 = [&](size_t off) { uint32_t v; memcpy(&v, b.data() + off, 4); return (uint64_t)v; };
  auto u64 = [&](size_t off) { uint64_t v; memcpy(&v, b.data() + off, 8); return v; };
  auto inside = [&](uint64_t off, uint64_t len) { return off <= n && len <= n - off; };
  const uint64_t phoff = u64(0x20), shoff = u64(0x28);
  const uint64_t phentsize = u16(0x36), phnum = u16(0x38), shentsize = u16(0x3a), shnum = u16(0x3c);
  if (!shnum || shentsize < 64 || !inside(shoff, shentsize * shnum)) return false;
  if (phnum && (phentsize < 56 || !inside(phoff, phentsize * phnum))) return false;
  for (uint64_t i = 0; i < shnum; ++i) {
    const size_t h = (size_t)(shoff + i * shentsize);
    if (u32(h + 4) == 8 /* SHT_NOBITS: no bytes in the file */) continue;
    if (!inside(u64(h + 0x18), u64(h + 0x20))) return false;
  }
  for (uint64_t i = 0; i < phnum; ++i) {
    const size_t h = (size_t)(phoff + i * phentsize);
    if (!inside(u64(h + 0x08), u64(h + 0x20))) return false;   // p_offset, p_filesz
  }
  return true;
}

int get_kernel(const std::string& source, const std::string& entry, Kernel* out) {
  std::lock_guard<std::mutex> lk(g_mu);
  const std::string arch = target_arch();
  const std::string h = source_hash(source, arch);
  const bool have_device = rt().ready;
  if (have_device) {
    auto it = g_kernels.find(h);
    if (it != g_kernels.end()) {
      ++g_n_mem;
      *out = it->second;
      return THX_OK;
    }
  }
  if (const char* dump = getenv("THX_DUMP_DIR")) {  // the generated source, named by its entry point
    mkdirs(dump);
    std::ofstream f(std::string(dump) + "/" + entry + ".hip");
    f << source;
  }
  std::vector<char> code;
  const std::string& dir = cache_dir();
  const std::string path = dir.empty() ? "" : dir + "/" + h + ".hsaco";
  Kernel k;
  if (!path.empty()) {
    std::ifstream f(path, std::ios::binary);
    if (f) {
      code.assign(std::istreambuf_iterator<char>(f), std::istreambuf_iterator<char>());
      // A cached file that is not a whole code object (cut short, overwritten), or one the device will
      // not load, is dropped and built again.
      bool good = !code.empty() && elf_complete(code);
      if (good && have_device &&
          (hipModuleLoadData(&k.module, code.data()) != hipSuccess ||
           hipModuleGetFunction(&k.func, k.module, entry.c_str()) != hipSuccess)) {
        (void)hipGetLastError();
        if (k.module) (void)hipModuleUnload(k.module);
        k = Kernel();
        good = false;
      }
      if (!good) {
        code.clear();
        unlink(path.c_str());
      }
      if (!code.empty()) ++g_n_disk;
    }
  }
  if (code.empty()) {
    int rc = compile_source(source, arch, &code);
    if (rc) return rc;
    ++g_n_compiled;
    if (!path.empty()) {
      mkdirs(dir);
      const std::string tmp = path + ".tmp" + std::to_string((long)getpid());
      std::ofstream f(tmp, std::ios::binary);
      if (f) {
        f.write(code.data(), (std::streamsize)code.size());
        f.close();
        if (!f || rename(tmp.c_str(), path.c_str()) != 0) unlink(tmp.c_str());   // a short write (disk full) is not kept
      }
    }
  }
  if (!have_device) {  // dry run: the code object is compiled and cached only
    *out = Kernel();
    return THX_OK;
  }
  if (!k.func) {
    THX_HIP_CHECK(hipModuleLoadData(&k.module, code.data()));
    hipError_t fe = hipModuleGetFunction(&k.func, k.module, entry.c_str());
    if (fe != hipSuccess) {
      (void)hipModuleUnload(k.module);
      return fail(THX_ERR_HIP, "hipModuleGetFunction(%s): %s", entry.c_str(), hipGetErrorString(fe));
    }
  }
  g_kernels[h] = k;
  *out = k;
  return THX_OK;
}

std::string entry_name(const std::string& functor, const std::string& plan) {
  std::string out = "thx_";
  for (char c : plan) out += (isalnum((unsigned char)c) ? c : '_');
  out += "_" + functor;
  return out;
}

int launch(const Kernel& k, const std::string& plan_in, unsigned grid, unsigned block, const void* params,
           size_t params_bytes, bool bare) {
  const std::string& plan = plan_in;
  if (!k.func) return fail(THX_ERR_HIP, "launch of '%s' without a loaded kernel", plan.c_str());
  if (params_bytes > 4096)
    return fail(THX_ERR_UNSUPPORTED, "kernel '%s' needs %zu bytes of arguments (limit 4096)", plan.c_str(),
                params_bytes);
  void* extra[] = {HIP_LAUNCH_PARAM_BUFFER_POINTER, const_cast<void*>(params), HIP_LAUNCH_PARAM_BUFFER_SIZE,
                   &params_bytes, HIP_LAUNCH_PARAM_END};
  Runtime& r = rt();
  if (!g_profiling || bare) {
    THX_HIP_CHECK(hipModuleLaunchKernel(k.func, grid, 1, 1, block, 1, 1, 0, r.stream, nullptr, extra));
    return THX_OK;
  }
  // Profiling: an event pair around the launch.  The elapsed time includes the events' own
  // processing (a few microseconds); a profiler's kernel trace gives the bare duration.
  ProfRec rec;
  rec.plan = plan;
  THX_HIP_CHECK(hipEventCreate(&rec.a));
  THX_HIP_CHECK(hipEventCreate(&rec.b));
  THX_HIP_CHECK(hipEventRecord(rec.a, r.stream));
  THX_HIP_CHECK(hipModuleLaunchKernel(k.func, grid, 1, 1, block, 1, 1, 0, r.stream, nullptr, extra));
  THX_HIP_CHECK(hipEventRecord(rec.b, r.stream));
  g_prof.push_back(rec);
  return THX_OK;
}

__global__ void thx_fill_kernel(unsigned char* dst, unsigned char value, size_t n) {
  const size_t stride = (size_t)gridDim.x * blockDim.x * 16;
  for (size_t i = ((size_t)blockIdx.x * blockDim.x + threadIdx.x) * 16; i < n; i += stride) {
    if (i + 16 <= n && (((uintptr_t)(dst + i)) & 15) == 0) {
      const unsigned w = value * 0x01010101u;
      *(uint4*)(dst + i) = make_uint4(w, w, w, w);
    } else {
      for (size_t j = i; j < n && j < i + 16; ++j) dst[j] = value;
    }
  }
}

}  // namespace thx

using namespace thx;

// ---------------------------------------------------------------------------
// C ABI
extern "C" {

const char* thx_last_error(void) { return g_error.c_str(); }
const char* thx_last_plan(void) { return g_plan.c_str(); }

int thx_init(int device) {
  std::lock_guard<std::mutex> lk(g_mu);
  return init_locked(device);
}

int thx_device_info(char* arch, size_t arch_cap, int* compute_units, int64_t* hbm_bytes) {
  int rc = ensure_init();
  if (rc) return rc;
  if (arch && arch_cap) snprintf(arch, arch_cap, "%s", rt().arch.c_str());
  if (compute_units) *compute_units = rt().cus;
  if (hbm_bytes) *hbm_bytes = rt().hbm;
  return THX_OK;
}

int thx_alloc(size_t nbytes, void** out) {
  int rc = ensure_init();
  if (rc) return rc;
  std::lock_guard<std::mutex> lk(g_mu);
  const size_t sz = nbytes ? (nbytes + 511) / 512 * 512 : 512;
  auto it = g_free.find(sz);
  if (it != g_free.end() && !it->second.empty()) {
    *out = it->second.back();
    it->second.pop_back();
    g_live[*out] = sz;
    return THX_OK;
  }
  void* p = nullptr;
  hipError_t e = hipMalloc(&p, sz);
  if (e != hipSuccess) {
    (void)hipGetLastError();
    (void)hipStreamSynchronize(rt().stream);
    for (auto& kv : g_free) {
      for (void* q : kv.second) (void)hipFree(q);
      kv.second.clear();
    }
    e = hipMalloc(&p, sz);
  }
  if (e != hipSuccess) {
    (void)hipGetLastError();
    return fail(THX_ERR_MEMORY, "device allocation of %zu bytes failed: %s", sz, hipGetErrorString(e));
  }
  g_live[p] = sz;
  *out = p;
  return THX_OK;
}

int thx_free(void* ptr) {
  if (!ptr) return THX_OK;
  std::lock_guard<std::mutex> lk(g_mu);
  auto it = g_live.find(ptr);
  if (it == g_live.end()) return fail(THX_ERR_ARG, "thx_free: %p was not allocated by thx_alloc", ptr);
  g_free[it->second].push_back(ptr);
  g_live.erase(it);
  return THX_OK;
}

int thx_pool_trim(void) {
  std::lock_guard<std::mutex> lk(g_mu);
  if (!rt().ready) return THX_OK;
  THX_HIP_CHECK(hipStreamSynchronize(rt().stream));
  for (auto& kv : g_free) {
    while (!kv.second.empty()) {
      void* q = kv.second.back();
      kv.second.pop_back();  // off the list before the call: a failed hipFree must not leave it to be handed out
      THX_HIP_CHECK(hipFree(q));
    }
  }
  return THX_OK;
}

int thx_h2d(void* dst, const void* src, size_t nbytes) {
  int rc = ensure_init();
  if (rc) return rc;
  if (!nbytes) return THX_OK;
  THX_HIP_CHECK(hipMemcpyAsync(dst, src, nbytes, hipMemcpyHostToDevice, rt().stream));
  THX_HIP_CHECK(hipStreamSynchronize(rt().stream));  // the host buffer may be pageable and reused at once
  return THX_OK;
}

int thx_d2h(void* dst, const void* src, size_t nbytes) {
  int rc = ensure_init();
  if (rc) return rc;
  if (!nbytes) return THX_OK;
  THX_HIP_CHECK(hipMemcpyAsync(dst, src, nbytes, hipMemcpyDeviceToHost, rt().stream));
  THX_HIP_CHECK(hipStreamSynchronize(rt().stream));
  return THX_OK;
}

int thx_d2d(void* dst, const void* src, size_t nbytes) {
  int rc = ensure_init();
  if (rc) return rc;
  if (!nbytes) return THX_OK;
  THX_HIP_CHECK(hipMemcpyAsync(dst, src, nbytes, hipMemcpyDeviceToDevice, rt().stream));
  return THX_OK;
}

int thx_fill_bytes(void* dst, int value, size_t nbytes) {
  int rc = ensure_init();
  if (rc) return rc;
  if (!nbytes) return THX_OK;
  size_t blocks = (nbytes / 16 + 255) / 256;
  if (blocks < 1) blocks = 1;
  if (blocks > 4096) blocks = 4096;
  hipLaunchKernelGGL(thx_fill_kernel, dim3((unsigned)blocks), dim3(256), 0, rt().stream, (unsigned char*)dst,
                     (unsigned char)value, nbytes);
  THX_HIP_CHECK(hipGetLastError());
  return THX_OK;
}

int thx_sync(void) {
  int rc = ensure_init();
  if (rc) return rc;
  THX_HIP_CHECK(hipStreamSynchronize(rt().stream));
  return THX_OK;
}

int thx_set_cache_dir(const char* path) {
  std::lock_guard<std::mutex> lk(g_mu);
  g_cache_dir = path ? path : "";
  g_cache_dir_set = true;
  return THX_OK;
}

int thx_cache_stats(int64_t* compiled, int64_t* disk_hits, int64_t* mem_hits) {
  std::lock_guard<std::mutex> lk(g_mu);
  if (compiled) *compiled = g_n_compiled;
  if (disk_hits) *disk_hits = g_n_disk;
  if (mem_hits) *mem_hits = g_n_mem;
  return THX_OK;
}

int thx_profile_begin(void) {
  int rc = ensure_init();
  if (rc) return rc;
  g_prof.clear();
  g_profiling = true;
  return THX_OK;
}

int thx_profile_end(char* buf, size_t cap) {
  if (!g_profiling) return fail(THX_ERR_ARG, "thx_profile_end without thx_profile_begin");
  g_profiling = false;
  THX_HIP_CHECK(hipStreamSynchronize(rt().stream));
  std::vector<std::string> order;
  std::unordered_map<std::string, std::pair<long, double>> agg;
  for (ProfRec& r : g_prof) {
    float ms = 0;
    THX_HIP_CHECK(hipEventElapsedTime(&ms, r.a, r.b));
    (void)hipEventDestroy(r.a);
    (void)hipEventDestroy(r.b);
    auto it = agg.find(r.plan);
    if (it == agg.end()) {
      order.push_back(r.plan);
      agg[r.plan] = {1, ms};
    } else {
      it->second.first += 1;
      it->second.second += ms;
    }
  }
  g_prof.clear();
  std::ostringstream os;
  for (const std::string& p : order) {
    char line[64];
    snprintf(line, sizeof line, "\t%ld\t%.6f\n", agg[p].first, agg[p].second);
    os << p << line;
  }
  const std::string s = os.str();
  if (s.size() + 1 > cap) return fail(THX_ERR_ARG, "thx_profile_end: buffer of %zu bytes, need %zu", cap, s.size() + 1);
  memcpy(buf, s.c_str(), s.size() + 1);
  return THX_OK;
}

int thx_timer_start(void) {
  int rc = ensure_init();
  if (rc) return rc;
  THX_HIP_CHECK(hipEventRecord(g_t0, rt().stream));
  return THX_OK;
}

int thx_timer_stop(float* elapsed_ms) {
  int rc = ensure_init();
  if (rc) return rc;
  THX_HIP_CHECK(hipEventRecord(g_t1, rt().stream));
  THX_HIP_CHECK(hipEventSynchronize(g_t1));
  THX_HIP_CHECK(hipEventElapsedTime(elapsed_ms, g_t0, g_t1));
  return THX_OK;
}

// ---- launch sequences recorded once and replayed (HIP graphs) ---------------------------------------------
struct thx_graph {
  hipGraph_t graph = nullptr;
  hipGraphExec_t exec = nullptr;
};

int thx_capture_begin(void) {
  int rc = ensure_init();
  if (rc) return rc;
  if (g_capturing) return fail(THX_ERR_ARG, "thx_capture_begin: a capture is already open");
  if (g_profiling) return fail(THX_ERR_ARG, "thx_capture_begin: not while profiling (its events are not part of the work)");
  THX_HIP_CHECK(hipStreamBeginCapture(rt().stream, hipStreamCaptureModeRelaxed));
  g_capturing = true;
  return THX_OK;
}

int thx_capture_end(thx_graph** out) {
  if (!g_capturing) return fail(THX_ERR_ARG, "thx_capture_end: no capture is open");
  g_capturing = false;
  hipGraph_t graph = nullptr;
  hipError_t e = hipStreamEndCapture(rt().stream, &graph);
  if (e != hipSuccess || !graph)
    return fail(THX_ERR_HIP, "hipStreamEndCapture failed: %s (a call that waits for the device ends a capture)",
                hipGetErrorString(e));
  if (!out) {                      // the caller only wanted to leave capture mode
    (void)hipGraphDestroy(graph);
    return THX_OK;
  }
  hipGraphExec_t exec = nullptr;
  e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
  if (e != hipSuccess) {
    (void)hipGraphDestroy(graph);
    return fail(THX_ERR_HIP, "hipGraphInstantiate failed: %s", hipGetErrorString(e));
  }
  thx_graph* g = new thx_graph;
  g->graph = graph;
  g->exec = exec;
  ++g_live_graphs;
  *out = g;
  return THX_OK;
}

int thx_graph_launch(thx_graph* g) {
  if (!g || !g->exec) return fail(THX_ERR_ARG, "thx_graph_launch: null graph");
  if (g_capturing) return fail(THX_ERR_ARG, "thx_graph_launch: a capture is open");
  THX_HIP_CHECK(hipGraphLaunch(g->exec, rt().stream));
  return THX_OK;
}

int thx_scratch_reserve(size_t nbytes) {
  int rc = ensure_init();
  if (rc) return rc;
  return ensure_scratch(nbytes);
}

int thx_scratch_state(int64_t* nbytes, int64_t* superseded_held, int64_t* graphs_alive) {
  if (nbytes) *nbytes = (int64_t)rt().scratch_bytes;
  if (superseded_held) *superseded_held = (int64_t)g_retired_scratch.size();
  if (graphs_alive) *graphs_alive = g_live_graphs;
  return THX_OK;
}

int thx_graph_free(thx_graph* g) {
  if (!g) return THX_OK;
  if (rt().ready) (void)hipStreamSynchronize(rt().stream);
  if (g->exec) (void)hipGraphExecDestroy(g->exec);
  if (g->graph) (void)hipGraphDestroy(g->graph);
  delete g;
  if (--g_live_graphs <= 0) {
    g_live_graphs = 0;
    release_retired_scratch();
  }
  return THX_OK;
}

}  // extern "C"
