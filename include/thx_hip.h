/*
 * thx_hip.h — C ABI of libthx_hip.so: fused Elemwise / CAReduce kernels for one
 * AMD MI355X (gfx950), compiled at run time with hipRTC.
 *
 * The library replaces, for Theano's data-parallel core, what the reference
 * reaches through pygpu / libgpuarray (citations are relative to the Theano
 * source tree):
 *   - GpuElemwise_new / GpuElemwise_call       theano/gpuarray/elemwise.py:240, 376
 *   - the generated GpuCAReduceCuda kernels and their launch code
 *                                              theano/gpuarray/elemwise.py:449-2420
 *   - pygpu_empty / GpuArray_write / GpuArray_read / GpuArray_memset
 *                                              theano/gpuarray/basic_ops.py:593-633, 708-741
 * Every function is plain C: pointers, sizes and PODs. All functions return
 * THX_OK (0) or an error code; thx_last_error() gives the message of the last
 * failure on the calling thread. One device, one in-order stream, no internal
 * threads. Device results are reproducible: values are never accumulated with
 * atomics (split reductions merge their partial results in a fixed order).  The
 * one atomic operation in the library counts arrivals: a split any / all
 * reduction adds its flags as 16-bit counts to a 64-bit word per result, and
 * counts do not depend on the order of arrival.
 */
#ifndef THX_HIP_H
#define THX_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define THX_MAX_ND 8

/* Error codes and the Python exception each one maps to (the classes raised by
 * the reference at theano/gpuarray/elemwise.py:292-315, 376-379, 642-654, 707-713). */
enum {
  THX_OK = 0,
  THX_ERR_HIP = 1,         /* RuntimeError: a HIP / hipRTC runtime call failed        */
  THX_ERR_SHAPE = 2,       /* ValueError:   input dimension mis-match                  */
  THX_ERR_TYPE = 3,        /* TypeError:    wrong rank, dtype or unusable strides      */
  THX_ERR_COMPILE = 4,     /* RuntimeError: hipRTC rejected generated source (log kept)*/
  THX_ERR_MEMORY = 5,      /* MemoryError:  device allocation failed                   */
  THX_ERR_UNSUPPORTED = 6, /* NotImplementedError                                     */
  THX_ERR_ARG = 7          /* ValueError:   malformed argument                         */
};

/* Element types; values are part of the ABI. */
enum {
  THX_BOOL = 0, THX_I8 = 1, THX_U8 = 2, THX_I16 = 3, THX_U16 = 4, THX_I32 = 5,
  THX_U32 = 6, THX_I64 = 7, THX_U64 = 8, THX_F16 = 9, THX_F32 = 10, THX_F64 = 11,
  THX_C64 = 12, THX_C128 = 13,   /* (real, imaginary) pairs of float32 / float64, NumPy's layout */
  THX_NDTYPES = 14
};

/* OR-ed into thx_array.dtype of an INPUT: `base + offset_bytes` is HOST memory
 * holding one element (all extents 1). Its value is copied into the kernel
 * arguments at call time, so it costs no device memory traffic. The reference
 * keeps 0-d operands on the host as well (theano/gpuarray/type.py:55-57).
 * Elements of up to 8 bytes only: a THX_C128 value goes through device memory. */
#define THX_HOST_SCALAR 0x100

/* OR-ed into thx_array.dtype (THX_I64, all extents 1, base ignored) of an input of
 * thx_reduce_call: a virtual operand whose value at an element is that element's
 * position within the reduced dimensions, counted in C order of those dimensions -
 * the index numpy.argmax returns after the reduced axes are moved to the end and
 * flattened, which is how MaxAndArgmax.perform defines its second output
 * (theano/tensor/basic.py:1311-1330). It costs no memory traffic. */
#define THX_INDEX 0x200

/* OR-ed into thx_array.dtype of an input or an output of a kernel call: one of the next calls reads
 * this array (again). It is then accessed with ordinary loads / stores, so that the 256 MB
 * last-level cache can serve the next read; arrays without the flag are streamed with
 * non-temporal accesses wherever that is the faster choice for the call. A hint only: results
 * never depend on it. */
#define THX_REUSED 0x400

/* A strided view of device memory (counterpart of libgpuarray's GpuArray:
 * data, offset, nd, dimensions, byte strides, typecode). Strides may be zero
 * or negative; they must be multiples of the element size. */
typedef struct thx_array {
  void* base;
  int64_t offset_bytes;
  int32_t nd;
  int32_t dtype;
  int64_t shape[THX_MAX_ND];
  int64_t strides_bytes[THX_MAX_ND];
} thx_array;

/* ---- device, memory, transfers ------------------------------------------ */

/* Select `device`, create the stream, read device properties. Idempotent. */
int thx_init(int device);
/* "gfx950:sramecc+:xnack-"-style architecture string and CU count of the device. */
int thx_device_info(char* arch, size_t arch_cap, int* compute_units, int64_t* hbm_bytes);
const char* thx_last_error(void);

/* Pooled device allocation (replaces pygpu_empty). thx_free returns the block
 * to the pool; thx_pool_trim releases cached blocks to the driver. */
int thx_alloc(size_t nbytes, void** out);
int thx_free(void* ptr);
int thx_pool_trim(void);
int thx_h2d(void* dst, const void* src, size_t nbytes);      /* GpuArray_write */
int thx_d2h(void* dst, const void* src, size_t nbytes);      /* GpuArray_read, synchronous */
int thx_d2d(void* dst, const void* src, size_t nbytes);
int thx_fill_bytes(void* dst, int value, size_t nbytes);     /* GpuArray_memset, a fill kernel */
int thx_sync(void);

/* ---- run-time compilation ----------------------------------------------- */

/* Directory of the on-disk code-object cache (default $THX_CACHE_DIR, else
 * ~/.cache/thx_hip). Pass NULL or "" to disable the disk cache. */
int thx_set_cache_dir(const char* path);
/* Counters since thx_init: kernels compiled by hipRTC, loaded from disk, and
 * served from memory. */
int thx_cache_stats(int64_t* compiled, int64_t* disk_hits, int64_t* mem_hits);

/* ---- Elemwise ------------------------------------------------------------ */

typedef struct thx_elemwise thx_elemwise;
typedef struct thx_reduce thx_reduce;

/* Create an n-ary elementwise operation from generated device source defining
 * a functor type named `functor_name` (see kernels/thx_elemwise.h for the
 * functor contract). Operands are the n_in inputs followed by the n_out
 * outputs; dtypes are THX_* codes in that order. Nothing is compiled yet:
 * kernels are specialised per access plan at the first call that needs them.
 * Replaces GpuElemwise_new (theano/gpuarray/elemwise.py:240). */
int thx_elemwise_new(const char* functor_src, const char* functor_name, int n_in, int n_out,
                     const int32_t* dtypes, thx_elemwise** out);

#define THX_BROADCAST 1 /* size-1 input dimensions broadcast against larger ones */
#define THX_DRY_RUN 2   /* validate, plan and compile (into the disk cache) but do not launch;
                           needs no device: the target is $THX_ARCH, default gfx950, and device
                           arrays may carry a null base (their addresses then count as aligned).
                           Without this flag an array that has elements and a null base is
                           refused with THX_ERR_ARG before anything is launched. */

/* Run on `ins` (n_in arrays) writing `outs` (n_out arrays, preallocated, every
 * one of the full result shape; an output may alias an input exactly for
 * in-place operation). All arrays must have the same rank (<= THX_MAX_ND).
 * The result shape is the broadcast of the inputs; where every input has
 * extent 1 the outputs' extent counts (a fill), and outputs may be strided
 * views (a copy into a slice of a larger array).
 * Fails with THX_ERR_SHAPE on a dimension mis-match. Asynchronous.
 * Replaces GpuElemwise_call(ge, args, GE_BROADCAST) (theano/gpuarray/elemwise.py:376). */
int thx_elemwise_call(thx_elemwise* e, const thx_array* ins, const thx_array* outs, int flags);
int thx_elemwise_free(thx_elemwise* e);

/* An elementwise result that is stored and also reduced over every dimension but the last (the
 * per-channel sum of an NHWC tensor that is an output as well): the reference runs GpuElemwise_call
 * and then a GpuCAReduceCuda kernel that reads the result back (theano/gpuarray/elemwise.py:376,
 * 1095-1723).  thx_elemwise_attach_reduce names the reduction `r` (created with thx_reduce_new,
 * no further epilogue operands) whose n_in inputs are the outputs which_outputs[0 .. n_in) of `e`;
 * the functor source given to thx_elemwise_new must then hold r's functor too and name it
 * (`typedef <r's functor> Red;` plus `red_lanes`, see kernels/thx_elemwise.h).
 * thx_elemwise_reduce_call = thx_elemwise_call plus that reduction into `red_outs` (C-contiguous,
 * one element per index of the last dimension): inside the same kernel where the access plan allows
 * it (permuted reads through LDS tiles), else by a reduction launched on the stored results.
 * Asynchronous; same error behaviour as thx_elemwise_call.
 * `e` borrows `r`: the reduction must stay alive until thx_elemwise_free(e) or until it is
 * detached with thx_elemwise_attach_reduce(e, NULL, NULL). */
int thx_elemwise_attach_reduce(thx_elemwise* e, thx_reduce* r, const int32_t* which_outputs);
int thx_elemwise_reduce_call(thx_elemwise* e, const thx_array* ins, const thx_array* outs,
                             const thx_array* red_outs, int flags);

/* ---- CAReduce ------------------------------------------------------------ */


/* Create a (multi-)reduction from generated device source defining a functor
 * named `functor_name` (contract in kernels/thx_reduce.h): n_in inputs feed a
 * fused prologue, n_out results of identical shape leave a fused epilogue that
 * may also read n_extra further operands (e.g. the divisor of a mean, a
 * per-channel scale). dtypes lists inputs, outputs, then those operands. acc_bytes = sizeof of the functor's
 * accumulator struct.
 * Replaces the kernel generation of GpuCAReduceCuda
 * (theano/gpuarray/elemwise.py:1756-2420). */
int thx_reduce_new(const char* functor_src, const char* functor_name, int n_in, int n_out, int n_extra,
                   const int32_t* dtypes, int acc_bytes, thx_reduce** out);

/* Reduce the dimensions d with reduce_mask[d] != 0. `ins` holds the n_in reduced
 * inputs, which all have rank nd and broadcast against each other like Elemwise
 * inputs, followed by the n_extra operands of the epilogue: each either a THX_HOST_SCALAR or a
 * device array with one element per result, laid out like a C-contiguous array with every stride
 * scaled by one factor (contiguous, or a view such as x[0, :, 0, 0]) and read at the result's
 * index; `outs` are
 * C-contiguous arrays of the kept dimensions, in order. A zero-length reduce domain yields
 * the identity (the caller rejects it for max/min, as
 * theano/tensor/elemwise.py:1489-1506 does). Asynchronous.
 * Replaces the c_code_reduce_* launch routines (theano/gpuarray/elemwise.py:1095-1723). */
int thx_reduce_call(thx_reduce* r, const thx_array* ins, const uint8_t* reduce_mask,
                    const thx_array* outs, int flags);

/* Size of the library's fixed scratch array, which every GPU the library runs on holds from the
 * moment the library is loaded until the process ends. */
#define THX_STATIC_SCRATCH_BYTES 4194304

/* thx_reduce_call for callers that cannot allocate device memory: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in
 * the reference.  Same arguments and results as thx_reduce_call, but the call never
 * allocates or frees device memory:
 *  - the partial results of a split reduction (S slices x results x accumulator bytes) go to the
 *    fixed scratch array instead of an allocated buffer; a reduction that needs more than
 *    THX_STATIC_SCRATCH_BYTES fails with THX_ERR_UNSUPPORTED and launches nothing;
 *  - compiling or loading a kernel allocates, so every kernel the call needs must already be
 *    loaded: run thx_reduce_call once on operands of the same layout beforehand (a warm-up);
 *    otherwise the call fails with THX_ERR_UNSUPPORTED and launches nothing;
 *  - thx_init must have been called (it resolves the array's device address); THX_DRY_RUN is
 *    refused; launches are never bracketed by profiling events.
 * Every call on a GPU shares that GPU's one array, which keeps the last call's contents: each
 * call overwrites every partial result before it reads it, so nothing needs clearing, but two
 * calls that overlap in time on one GPU (from different streams or threads) race.  Calls on the
 * library's one in-order stream never overlap. */
int thx_reduce_call_static(thx_reduce* r, const thx_array* ins, const uint8_t* reduce_mask,
                           const thx_array* outs, int flags);
int thx_reduce_free(thx_reduce* r);

/* ---- Row chains ------------------------------------------------------------ */

typedef struct thx_rowchain thx_rowchain;

/* Operand kinds of a row chain. */
enum { THX_KIND_FULL = 0, THX_KIND_ROW = 1, THX_KIND_COL = 2, THX_KIND_SCALAR = 3 };

/* Create a fused "elementwise + reductions along the last axis" operation from
 * generated device source defining a functor named `functor_name` (contract in
 * kernels/thx_rowchain.h). kinds[i] says how operand i (inputs, then outputs)
 * relates to the full shape [rows..., C]: FULL = that shape, ROW = one value
 * per row ([rows..., 1] or [rows...]), COL = one value per column ([1..., C]),
 * SCALAR = one value (device array or THX_HOST_SCALAR). Outputs are FULL or ROW.
 * The reference has no such kernel for arbitrary graphs; it covers row softmax
 * with the dedicated GpuSoftmax kernel (theano/gpuarray/nnet.py) instead. */
int thx_rowchain_new(const char* functor_src, const char* functor_name, int n_in, int n_out,
                     const int32_t* dtypes, const int32_t* kinds, thx_rowchain** out);
/* One launch: each row is read once, kept in registers through every step and
 * written once. Fails with THX_ERR_UNSUPPORTED - the caller then runs the
 * unfused nodes - when rows are not unit-stride, leading dimensions do not
 * collapse to one row stride, or a row exceeds 16384 vector slots. */
int thx_rowchain_call(thx_rowchain* c, const thx_array* ins, const thx_array* outs, int flags);
/* Reductions of the chain run over `axes` of the full shape instead of its last axis: reduced axes
 * may lie before and after one run of adjacent kept axes (axes (0, 2, 3) of [N, C, H, W] keep C, the
 * batch-normalisation statistics of theano/tensor/nnet/bn.py:364-760), and at least one must trail
 * them. ROW operands then hold one value per kept index (extent 1 on every reduced axis, or the
 * kept axes alone); COL operands are not taken. Such chains run in the held form only (one block per
 * kept index keeps that index's whole reduce domain on chip, kernels/thx_rowchain.h), which
 * thx_rowchain_call refuses with THX_ERR_UNSUPPORTED when a reduce domain exceeds what one compute
 * unit's registers and LDS hold or when there are too few kept indices to occupy the device. */
int thx_rowchain_set_axes(thx_rowchain* c, int n_axes, const int32_t* axes);
int thx_rowchain_free(thx_rowchain* c);

/* ---- inspection and timing ------------------------------------------------ */

/* Name of the kernel plan used by the last elemwise / reduce call on this
 * thread (e.g. "ew|nd1|i32|v4|u4|m0,1,1,0"), for tests and profiling. */
const char* thx_last_plan(void);

/* Per-kernel timing with HIP events on the library's stream. Between
 * thx_profile_begin and thx_profile_end every launch is bracketed by an event
 * pair; thx_profile_end synchronises and writes one line per kernel:
 * "<plan>\t<launches>\t<total_ms>\n". Returns THX_ERR_ARG if `cap` is too small. */
int thx_profile_begin(void);
int thx_profile_end(char* buf, size_t cap);

/* ---- recorded launch sequences -------------------------------------------
 * No counterpart in the reference (every GpuElemwise / GpuCAReduceCuda call is
 * launched on its own, theano/gpuarray/elemwise.py:376, :1095-1723).  For hosts
 * whose per-launch cost exceeds the kernels' run time: everything the library
 * launches between thx_capture_begin and thx_capture_end is recorded into a HIP
 * graph instead of run; thx_graph_launch replays it on the library's stream with
 * the very same addresses, so the caller keeps every array that took part alive
 * and unmoved until thx_graph_free.  Calls that wait for the device (thx_d2h,
 * thx_h2d, thx_sync, thx_timer_stop, thx_profile_*) must not be made while a
 * capture is open; run the sequence once before capturing it, so that kernels
 * are loaded and the allocation pool is warm.  thx_capture_end(NULL) abandons
 * the recording. */
typedef struct thx_graph thx_graph;
int thx_capture_begin(void);
int thx_capture_end(thx_graph** out);
int thx_graph_launch(thx_graph* g);
int thx_graph_free(thx_graph* g);

/* Partial results of split reductions live in one scratch buffer that grows on demand (8 MiB at
 * first).  While a recorded sequence is alive the buffer it was recorded with is kept, also after
 * a later call has needed a larger one; growing it inside a recording is refused.
 * thx_scratch_reserve sizes the buffer up-front; thx_scratch_state reports the current size, the
 * number of superseded buffers still held for recorded sequences, and the recorded sequences alive.
 * No counterpart in the reference (its reductions take no workspace). */
int thx_scratch_reserve(size_t nbytes);
int thx_scratch_state(int64_t* nbytes, int64_t* superseded_held, int64_t* graphs_alive);

/* Whole-region timing: events recorded on the library's stream. */
int thx_timer_start(void);
int thx_timer_stop(float* elapsed_ms); /* synchronises */

#ifdef __cplusplus
}
#endif
#endif /* THX_HIP_H */
