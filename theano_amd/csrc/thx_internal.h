// Host-side internals of libthx_hip.so shared by the runtime, the elementwise
// planner and the reduction planner.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>
#include <string>
#include <unordered_map>
#include <vector>

#include "../../include/thx_hip.h"

#define THX_TICKET_WORDS 4096

namespace thx {

// ---- errors ---------------------------------------------------------------
int fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));
void set_last_plan(const std::string& plan);
// True when `a` has elements and no address to read them at: such an operand must be refused before a
// kernel or a host copy dereferences it.  A dry run launches nothing and needs no device addresses; a scalar
// passed from the host is read by the planner itself and always needs one.
inline bool null_base(const thx_array& a, bool dry) {
  if (a.base || (a.dtype & THX_INDEX)) return false;
  if (dry && !(a.dtype & THX_HOST_SCALAR)) return false;
  for (int d = 0; d < a.nd && d < THX_MAX_ND; ++d)
    if (a.shape[d] == 0) return false;
  return true;
}

#define THX_HIP_CHECK(expr)                                                        \
  do {                                                                             \
    hipError_t e_ = (expr);                                                        \
    if (e_ != hipSuccess)                                                          \
      return ::thx::fail(THX_ERR_HIP, "%s failed: %s", #expr, hipGetErrorString(e_)); \
  } while (0)

// ---- global state -----------------------------------------------------------
struct Runtime {
  bool ready = false;
  int device = -1;
  int cus = 0;
  int64_t hbm = 0;
  std::string arch;       // as reported, e.g. gfx950:sramecc+:xnack-
  std::string arch_base;  // gfx950
  hipStream_t stream = nullptr;
  char* scratch = nullptr;  // partial results of split reductions
  size_t scratch_bytes = 0;
  // Device address of the library's fixed scratch array on `device` (thx_reduce_call_static),
  // resolved once in thx_init; null until then.
  char* static_scratch = nullptr;
  // Device address of THX_TICKET_WORDS zero words for reductions that finish with one atomic add per slice.
  char* ticket_words = nullptr;
};
Runtime& rt();
int ensure_init();
int ensure_scratch(size_t bytes);

// ---- run-time compilation ---------------------------------------------------
struct Kernel {
  hipModule_t module = nullptr;
  hipFunction_t func = nullptr;
};
// Compile (or fetch from the caches) `source`, which must define an
// extern "C" __global__ function named `entry`.
int get_kernel(const std::string& source, const std::string& entry, Kernel* out);
// True (default; $THX_FAST_DIV=0 turns it off) when float32 division / sqrt are compiled to the 2.5-ulp forms.
bool fast_div();
// Non-temporal accesses: $THX_NT when set, else the default of the kernel family (measured per family).
int nt_choice(int family_default);
// Elementwise and row-chain kernels: non-temporal when the operands together (`moved` bytes) exceed
// what the 256 MB last-level cache can keep for a consumer; measured on inputs that are not cached,
// non-temporal accesses are 4-8% faster from about 300 MB up and 2-3% slower below.
int nt_streaming(int64_t moved);
// The embedded device headers (thx_common.h, thx_elemwise.h, thx_reduce.h).
const std::string& device_prelude();

// Kernel symbol for a plan: "thx_" + plan with punctuation folded to '_' + "_" + functor, so that
// profilers show one line per (functor, plan) instead of a shared entry name.
std::string entry_name(const std::string& functor, const std::string& plan);

// Launch with one by-value parameter block.  `bare`: never bracket the launch with profiling
// events (creating an event allocates; callers that must not allocate pass true).
int launch(const Kernel& k, const std::string& plan, unsigned grid, unsigned block,
           const void* params, size_t params_bytes, bool bare = false);

// ---- array helpers ----------------------------------------------------------
int dtype_size(int dtype);
const char* dtype_ctype(int dtype);

// FastDiv as laid out in kernels/thx_common.h.
struct FastDivH {
  uint32_t m, s, d, pad;
};
FastDivH make_fastdiv(uint64_t d);

// Byte-wise builder for kernel parameter blocks whose layout depends on
// template arguments; mirrors the natural alignment rules of the device structs.
struct ParamPack {
  std::vector<unsigned char> buf;
  void align(size_t a) {
    while (buf.size() % a) buf.push_back(0);
  }
  template <class T>
  void put(const T& v) {
    align(alignof(T));
    const unsigned char* p = reinterpret_cast<const unsigned char*>(&v);
    buf.insert(buf.end(), p, p + sizeof(T));
  }
  void put_index(bool wide, int64_t v) {
    if (wide) put<int64_t>(v);
    else put<int32_t>(static_cast<int32_t>(v));
  }
};

// One operand after validation: element strides over the common shape.
struct View {
  char* ptr = nullptr;
  int dtype = 0;
  bool imm = false;     // a host scalar travelling in the kernel arguments
  uint64_t immval = 0;  // its value bytes
  bool iota = false;    // no memory: the strides are index multipliers and the value is the offset
  bool reused = false;  // THX_REUSED: a later call reads it, keep it cacheable
  int64_t stride[THX_MAX_ND] = {0};
};

// Bit mask over operands: the call-wide choice `nt`, withdrawn from operands flagged THX_REUSED
// (unless $THX_NT forces it).
uint64_t nt_mask(int nt, const std::vector<View>& views);

// Check ranks/dtypes, compute the broadcast shape of `ins`, convert strides to
// elements (0 on broadcast dimensions). `what` names the operation in messages.
int gather_inputs(const char* what, const thx_array* ins, int n_in, const int32_t* dtypes, int flags,
                  int* nd_out, int64_t* shape, std::vector<View>* views);

}  // namespace thx

// ---- operation handles --------------------------------------------------------
struct thx_reduce {
  std::string src, name;
  int n_in = 0, n_out = 0, n_extra = 0, acc_bytes = 0;
  std::vector<int32_t> dtypes;
  std::unordered_map<std::string, thx::Kernel> plans;
  bool has_ticket = false;  // the functor packs its accumulators into counts (ticket_pack / ticket_unpack)
};

struct thx_elemwise {
  std::string src, name;
  int n_in = 0, n_out = 0;
  std::vector<int32_t> dtypes;
  std::unordered_map<std::string, thx::Kernel> plans;
  // the reduction attached by thx_elemwise_attach_reduce: its inputs are the outputs red_of[0..] of this operation
  thx_reduce* red = nullptr;
  std::vector<int32_t> red_of;
};

namespace thx {
// Second pass of a split reduction (merges S partial accumulators per result in slice order and runs the
// epilogue); S = 0 writes the identity through the epilogue.  `fixed`: nothing that allocates.
int reduce_final_pass(thx_reduce* r, const std::vector<char*>& outp, const std::vector<uint64_t>& ex,
                      const std::vector<int64_t>& exs, char* partial, int64_t n_out, int S, bool dry, bool fixed);
}  // namespace thx
