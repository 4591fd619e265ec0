/*
 * TEST INFRASTRUCTURE - not part of the product. Only tests/, bench.py's
 * cpu_baseline leg and __graft_entry__.smoke() may load this.
 *
 * CPU restatement of Theano's C backend for CAReduce
 * (theano/tensor/elemwise.py:1384-1556 with the loop nest of
 * theano/tensor/elemwise_cgen.py:465-527):
 *   - loop order: kept dimensions (ascending) outermost, reduced dimensions
 *     (ascending) innermost                         elemwise.py:1419-1420
 *   - one accumulator of acc_dtype per output, set to the identity when the
 *     reduced loops start                           elemwise.py:1536-1542
 *   - inner statement acc = scalar_op(acc, x) with C's usual conversions
 *                                                   elemwise.py:1511-1533
 *   - strictly sequential and single-threaded: make_loop_careduce emits no
 *     OpenMP pragma.
 * The accumulator array is returned; the final cast to the output dtype
 * (PyArray_CopyInto, elemwise.py:1549-1554) is done by the caller.
 * Per-op expressions follow theano/scalar/basic.py: Add :1707-1716,
 * Mul :1752-1761, Maximum :1632-1639, Minimum :1669-1675, OR/XOR/AND
 * :1561-1600 (bool add/mul are || and &&); mul_without_zeros
 * theano/tensor/elemwise.py:2072-2077 (identity 0).
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

enum { OP_ADD = 0, OP_MUL = 1, OP_MAX = 2, OP_MIN = 3, OP_AND = 4, OP_OR = 5, OP_XOR = 6, OP_MULNZ = 7 };
enum { T_BOOL = 0, T_I8, T_U8, T_I16, T_U16, T_I32, T_U32, T_I64, T_U64, T_F16, T_F32, T_F64 };

#define MAXND 16

typedef struct {
  int nk, nr;
  int64_t kshape[MAXND], kstride[MAXND], rshape[MAXND], rstride[MAXND];
} plan_t;

/* Walks the reduce domain of one output in row-major order of the reduced
 * dimensions, the innermost one as a tight strided loop. */
#define DEFINE_REDUCE(NAME, IN_T, ACC_T, STMT)                                               \
  static void NAME(const plan_t* p, const char* base, ACC_T* accp) {                         \
    ACC_T acc = *accp;                                                                       \
    int64_t idx[MAXND];                                                                      \
    const int nr = p->nr;                                                                    \
    if (nr == 0) {                                                                           \
      const IN_T x = *(const IN_T*)base;                                                     \
      STMT;                                                                                  \
      *accp = acc;                                                                           \
      return;                                                                                \
    }                                                                                        \
    for (int d = 0; d < nr; ++d) idx[d] = 0;                                                 \
    const int64_t n_in = p->rshape[nr - 1], s_in = p->rstride[nr - 1];                       \
    for (;;) {                                                                               \
      const char* q = base;                                                                  \
      for (int d = 0; d < nr - 1; ++d) q += idx[d] * p->rstride[d];                          \
      for (int64_t i = 0; i < n_in; ++i) {                                                   \
        const IN_T x = *(const IN_T*)(q + i * s_in);                                         \
        STMT;                                                                                \
      }                                                                                      \
      int d = nr - 2;                                                                        \
      while (d >= 0 && ++idx[d] == p->rshape[d]) idx[d--] = 0;                               \
      if (d < 0) break;                                                                      \
    }                                                                                        \
    *accp = acc;                                                                             \
  }

#define MAXSTMT acc = ((x) > (acc) ? (x) : ((acc) >= (x) ? (acc) : nan("")))
#define MINSTMT acc = ((x) < (acc) ? (x) : ((acc) <= (x) ? (acc) : nan("")))
#define IMAXSTMT acc = ((x) > (acc) ? (x) : (acc))
#define IMINSTMT acc = ((x) < (acc) ? (x) : (acc))

/* sums and products: (in, acc) pairs of theano/tensor/elemwise.py:1746-1759 plus acc == in */
#define SUMPROD(IN_N, IN_T, ACC_N, ACC_T)                                  \
  DEFINE_REDUCE(add_##IN_N##_##ACC_N, IN_T, ACC_T, acc = acc + x)          \
  DEFINE_REDUCE(mul_##IN_N##_##ACC_N, IN_T, ACC_T, acc = acc * x)

/* every input type with every accumulator type a caller may ask for (acc_dtype=..., elemwise.py:1760-1780);
 * float16 inputs arrive converted to float32, bool and float16 accumulators have no C code */
#define SUMPROD_INTO(ACC_N, ACC_T)       \
  SUMPROD(bool, uint8_t, ACC_N, ACC_T)   \
  SUMPROD(i8, int8_t, ACC_N, ACC_T)      \
  SUMPROD(u8, uint8_t, ACC_N, ACC_T)     \
  SUMPROD(i16, int16_t, ACC_N, ACC_T)    \
  SUMPROD(u16, uint16_t, ACC_N, ACC_T)   \
  SUMPROD(i32, int32_t, ACC_N, ACC_T)    \
  SUMPROD(u32, uint32_t, ACC_N, ACC_T)   \
  SUMPROD(i64, int64_t, ACC_N, ACC_T)    \
  SUMPROD(u64, uint64_t, ACC_N, ACC_T)   \
  SUMPROD(f32, float, ACC_N, ACC_T)      \
  SUMPROD(f64, double, ACC_N, ACC_T)
SUMPROD_INTO(i8, int8_t)
SUMPROD_INTO(u8, uint8_t)
SUMPROD_INTO(i16, int16_t)
SUMPROD_INTO(u16, uint16_t)
SUMPROD_INTO(i32, int32_t)
SUMPROD_INTO(u32, uint32_t)
SUMPROD_INTO(i64, int64_t)
SUMPROD_INTO(u64, uint64_t)
SUMPROD_INTO(f32, float)
SUMPROD_INTO(f64, double)

/* theano/tensor/elemwise.py:2075-2077 with x = accumulator, y = element */
#define MULNZSTMT acc = ((acc == 0) ? (x) : (((x) == 0) ? (acc) : ((x) * (acc))))
DEFINE_REDUCE(mulnz_f32_f64, float, double, MULNZSTMT)
DEFINE_REDUCE(mulnz_f32_f32, float, float, MULNZSTMT)
DEFINE_REDUCE(mulnz_f64_f64, double, double, MULNZSTMT)

#define MAXMIN_F(N, T)                           \
  DEFINE_REDUCE(max_##N##_##N, T, T, MAXSTMT)    \
  DEFINE_REDUCE(min_##N##_##N, T, T, MINSTMT)
#define MAXMIN_I(N, T)                           \
  DEFINE_REDUCE(max_##N##_##N, T, T, IMAXSTMT)   \
  DEFINE_REDUCE(min_##N##_##N, T, T, IMINSTMT)
MAXMIN_F(f32, float)
MAXMIN_F(f64, double)
MAXMIN_I(bool, uint8_t)
MAXMIN_I(i8, int8_t)
MAXMIN_I(u8, uint8_t)
MAXMIN_I(i16, int16_t)
MAXMIN_I(u16, uint16_t)
MAXMIN_I(i32, int32_t)
MAXMIN_I(u32, uint32_t)
MAXMIN_I(i64, int64_t)
MAXMIN_I(u64, uint64_t)

#define BITOPS(N, T)                                        \
  DEFINE_REDUCE(and_##N##_##N, T, T, acc = (acc & x))       \
  DEFINE_REDUCE(or_##N##_##N, T, T, acc = (acc | x))        \
  DEFINE_REDUCE(xor_##N##_##N, T, T, acc = (acc ^ x))
BITOPS(bool, uint8_t)
BITOPS(i8, int8_t)
BITOPS(u8, uint8_t)
BITOPS(i16, int16_t)
BITOPS(u16, uint16_t)
BITOPS(i32, int32_t)
BITOPS(u32, uint32_t)
BITOPS(i64, int64_t)
BITOPS(u64, uint64_t)

typedef void (*reduce_fn)(const plan_t*, const char*, void*);

typedef struct {
  int op, in, acc;
  reduce_fn fn;
} entry_t;

#define E(OP, IN, ACC, NAME) {OP, IN, ACC, (reduce_fn)NAME}
#define ESP(INC, INN, ACCC, ACCN) E(OP_ADD, INC, ACCC, add_##INN##_##ACCN), E(OP_MUL, INC, ACCC, mul_##INN##_##ACCN)
#define ESP_INTO(ACCC, ACCN)                                                                                   \
  ESP(T_BOOL, bool, ACCC, ACCN), ESP(T_I8, i8, ACCC, ACCN), ESP(T_U8, u8, ACCC, ACCN), ESP(T_I16, i16, ACCC, ACCN),  \
      ESP(T_U16, u16, ACCC, ACCN), ESP(T_I32, i32, ACCC, ACCN), ESP(T_U32, u32, ACCC, ACCN),                     \
      ESP(T_I64, i64, ACCC, ACCN), ESP(T_U64, u64, ACCC, ACCN), ESP(T_F32, f32, ACCC, ACCN),                     \
      ESP(T_F64, f64, ACCC, ACCN)
#define EMM(C, N) E(OP_MAX, C, C, max_##N##_##N), E(OP_MIN, C, C, min_##N##_##N)
#define EBIT(C, N) E(OP_AND, C, C, and_##N##_##N), E(OP_OR, C, C, or_##N##_##N), E(OP_XOR, C, C, xor_##N##_##N)

static const entry_t table[] = {
    ESP_INTO(T_I8, i8),   ESP_INTO(T_U8, u8),   ESP_INTO(T_I16, i16), ESP_INTO(T_U16, u16), ESP_INTO(T_I32, i32),
    ESP_INTO(T_U32, u32), ESP_INTO(T_I64, i64), ESP_INTO(T_U64, u64), ESP_INTO(T_F32, f32), ESP_INTO(T_F64, f64),
    EMM(T_F32, f32),  EMM(T_F64, f64),  EMM(T_BOOL, bool), EMM(T_I8, i8),   EMM(T_U8, u8),   EMM(T_I16, i16),
    EMM(T_U16, u16),  EMM(T_I32, i32),  EMM(T_U32, u32),   EMM(T_I64, i64), EMM(T_U64, u64),
    EBIT(T_BOOL, bool), EBIT(T_I8, i8), EBIT(T_U8, u8), EBIT(T_I16, i16), EBIT(T_U16, u16), EBIT(T_I32, i32),
    EBIT(T_U32, u32),   EBIT(T_I64, i64), EBIT(T_U64, u64),
    E(OP_MULNZ, T_F32, T_F64, mulnz_f32_f64), E(OP_MULNZ, T_F32, T_F32, mulnz_f32_f32),
    E(OP_MULNZ, T_F64, T_F64, mulnz_f64_f64),
};

static int tsize(int t) {
  static const int s[] = {1, 1, 1, 2, 2, 4, 4, 8, 8, 2, 4, 8};
  return s[t];
}

/* Returns 0, or -1 when the (op, in, acc) combination is not restated here.
 * `identity` points to one value of acc_dtype; `out` receives one acc_dtype
 * value per output, C-contiguous over the kept dimensions. */
int oracle_careduce(int op, int in_dtype, int acc_dtype, int nd, const int64_t* shape, const int64_t* strides_bytes,
                    const uint8_t* mask, const void* in, const void* identity, void* out) {
  reduce_fn fn = 0;
  for (unsigned i = 0; i < sizeof table / sizeof table[0]; ++i)
    if (table[i].op == op && table[i].in == in_dtype && table[i].acc == acc_dtype) fn = table[i].fn;
  if (!fn || nd > MAXND) return -1;
  plan_t p;
  p.nk = p.nr = 0;
  int64_t n_out = 1, n_red = 1;
  for (int d = 0; d < nd; ++d) {
    if (mask[d]) {
      p.rshape[p.nr] = shape[d];
      p.rstride[p.nr++] = strides_bytes[d];
      n_red *= shape[d];
    } else {
      p.kshape[p.nk] = shape[d];
      p.kstride[p.nk++] = strides_bytes[d];
      n_out *= shape[d];
    }
  }
  const int asz = tsize(acc_dtype);
  int64_t idx[MAXND];
  for (int d = 0; d < p.nk; ++d) idx[d] = 0;
  for (int64_t o = 0; o < n_out; ++o) {
    char* dst = (char*)out + o * asz;
    memcpy(dst, identity, (size_t)asz);
    if (n_red > 0) {
      const char* base = (const char*)in;
      for (int d = 0; d < p.nk; ++d) base += idx[d] * p.kstride[d];
      fn(&p, base, dst);
    }
    int d = p.nk - 1;
    while (d >= 0 && ++idx[d] == p.kshape[d]) idx[d--] = 0;
  }
  return 0;
}
