/*
 * sort_oracle.c -- TEST INFRASTRUCTURE, not part of the product.
 *
 * Plain-C restatement of the single-processor CPU/OpenMP variant of cuPyNumeric's SORT task,
 * used only as the checker in tests/, by __graft_entry__.smoke() and as the timed
 * `cpu_baseline` of bench.py.  Nothing under cupynumeric_amd/ calls it.
 *
 * What it follows in the reference (/root/reference):
 *   SortImplBodyCpu            src/cupynumeric/sort/sort_cpu.inl:937-1074
 *       key copy for argsort   :974-976      index init  :990-1002 (sort.h:83-92: i % seg + offset)
 *       copy input -> output   :1022-1025    then the in-place local sort :1026
 *   thrust_local_sort_inplace  src/cupynumeric/sort/sort_cpu.inl:52-85
 *       serial loop over segments, each thrust::(stable_)sort[_by_key](exec, ..., less)
 *       exec = thrust::host (sort.cc:64)  or  thrust::omp::par (sort_omp.cc:65): the threads
 *       work inside one segment, the segment loop stays serial.
 *
 * thrust itself (CCCL, pulled in through Legate; not under /root/reference) is not restated:
 * the per-segment sort is a textbook stable merge sort.  Its comparison is NumPy's order --
 * integers by value, floats ascending with every NaN last and -0.0 == +0.0, complex numbers by
 * (real, imag) with NaNs last -- which is the
 * ordering contract of this build; thrust's own treatment of NaN (unordered under `less`,
 * bit-pattern order under its host radix sort) is deliberately not reproduced.  Unstable
 * kinds are served by the same stable sort (any stable result is a valid unstable one).
 *
 * Parity pins (tests/test_oracle.py): the golden vectors of the reference's own tests
 * (tests/cpp/integration/test_sort.cc, test_argsort.cc), NumPy's independent stable sort,
 * closed forms (reversed, all-equal, inverse permutation) and a brute-force insertion sort
 * over a NaN / +-0 / inf alphabet.
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

/* element type codes: same values as enum cpn_dtype in include/cpn_sort.h */
enum { T_BOOL, T_I8, T_I16, T_I32, T_I64, T_U8, T_U16, T_U32, T_U64, T_F16, T_F32, T_F64, T_C64, T_C128 };

/* ---- NumPy's "less" for floating point: a < b, or b is NaN and a is not ---------------- */
static inline int less_f32(float a, float b) { return a < b || (b != b && a == a); }
static inline int less_f64(double a, double b) { return a < b || (b != b && a == a); }

/* IEEE binary16 bits -> float (exact) */
static inline float half_to_float(uint16_t h)
{
  const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  const uint32_t exp  = (h >> 10) & 0x1Fu;
  uint32_t man        = h & 0x3FFu;
  uint32_t bits;
  if (exp == 0) {
    if (man == 0) {
      bits = sign;
    } else { /* subnormal: normalise */
      int e = -1;
      do {
        man <<= 1;
        ++e;
      } while ((man & 0x400u) == 0);
      bits = sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3FFu) << 13);
    }
  } else if (exp == 31) {
    bits = sign | 0x7F800000u | (man << 13);
  } else {
    bits = sign | ((exp + 127 - 15) << 23) | (man << 13);
  }
  float f;
  memcpy(&f, &bits, 4);
  return f;
}
static inline int less_f16(uint16_t a, uint16_t b) { return less_f32(half_to_float(a), half_to_float(b)); }

/*
 * Complex numbers: NumPy's order (numpy/_core/src/npysort/npysort_common.h, CFLOAT_LT /
 * CDOUBLE_LT), restated branch for branch: lexicographic on (real, imag) with NaNs last.  The
 * reference compares complex values with thrust and `less` on legate::Complex
 * (src/cupynumeric/sort/thrust_sort.h:129-145), which agrees on NaN-free data (the only data
 * its tests feed, tests/cpp/integration/test_sort.cc:98-134).
 */
typedef struct { float re, im; } c64_t;
typedef struct { double re, im; } c128_t;
#define DEFINE_CLT(NAME, T)                                                            \
  static inline int NAME(T a, T b)                                                     \
  {                                                                                    \
    if (a.re < b.re) {                                                                 \
      return a.im == a.im || b.im != b.im;                                             \
    } else if (a.re > b.re) {                                                          \
      return b.im != b.im && a.im == a.im;                                             \
    } else if (a.re == b.re || (a.re != a.re && b.re != b.re)) {                       \
      return a.im < b.im || (b.im != b.im && a.im == a.im);                            \
    } else {                                                                           \
      return b.re != b.re;                                                             \
    }                                                                                  \
  }
DEFINE_CLT(less_c64, c64_t)
DEFINE_CLT(less_c128, c128_t)

#define LESS_INT(a, b) ((a) < (b))

/*
 * Stable merge sort of keys[0..n) carrying idx (may be NULL), scratch tk/ti of n elements.
 * Runs of RUN elements by insertion sort, then bottom-up merging.  With OpenMP the segment
 * is cut into one block per thread, blocks are sorted concurrently and merged pairwise.
 */
#define RUN 24

#define DEFINE_SORT(NAME, T, LESS)                                                               \
  static void NAME##_insertion(T* k, int64_t* ix, size_t n)                                      \
  {                                                                                              \
    for (size_t i = 1; i < n; ++i) {                                                             \
      const T v       = k[i];                                                                    \
      const int64_t w = ix ? ix[i] : 0;                                                          \
      size_t j        = i;                                                                       \
      while (j > 0 && LESS(v, k[j - 1])) {                                                       \
        k[j] = k[j - 1];                                                                         \
        if (ix) ix[j] = ix[j - 1];                                                               \
        --j;                                                                                     \
      }                                                                                          \
      k[j] = v;                                                                                  \
      if (ix) ix[j] = w;                                                                         \
    }                                                                                            \
  }                                                                                              \
  /* merge [lo,mid) and [mid,hi) of (sk,si) into (dk,di); ties take the left run first */        \
  static void NAME##_merge(const T* sk, const int64_t* si, T* dk, int64_t* di, size_t lo,        \
                           size_t mid, size_t hi)                                                \
  {                                                                                              \
    size_t a = lo, b = mid, o = lo;                                                              \
    while (a < mid && b < hi) {                                                                  \
      if (LESS(sk[b], sk[a])) {                                                                  \
        dk[o] = sk[b];                                                                           \
        if (si) di[o] = si[b];                                                                   \
        ++b;                                                                                     \
      } else {                                                                                   \
        dk[o] = sk[a];                                                                           \
        if (si) di[o] = si[a];                                                                   \
        ++a;                                                                                     \
      }                                                                                          \
      ++o;                                                                                       \
    }                                                                                            \
    while (a < mid) {                                                                            \
      dk[o] = sk[a];                                                                             \
      if (si) di[o] = si[a];                                                                     \
      ++a;                                                                                       \
      ++o;                                                                                       \
    }                                                                                            \
    while (b < hi) {                                                                             \
      dk[o] = sk[b];                                                                             \
      if (si) di[o] = si[b];                                                                     \
      ++b;                                                                                       \
      ++o;                                                                                       \
    }                                                                                            \
  }                                                                                              \
  /* sequential stable sort of one block; result ends in (k, ix) */                              \
  static void NAME##_block(T* k, int64_t* ix, T* tk, int64_t* ti, size_t n)                      \
  {                                                                                              \
    for (size_t s = 0; s < n; s += RUN) {                                                        \
      const size_t len = (n - s < RUN) ? n - s : RUN;                                            \
      NAME##_insertion(k + s, ix ? ix + s : NULL, len);                                          \
    }                                                                                            \
    T* sk       = k;                                                                             \
    int64_t* si = ix;                                                                            \
    T* dk       = tk;                                                                            \
    int64_t* di = ti;                                                                            \
    for (size_t w = RUN; w < n; w *= 2) {                                                        \
      for (size_t lo = 0; lo < n; lo += 2 * w) {                                                 \
        const size_t mid = (lo + w < n) ? lo + w : n;                                            \
        const size_t hi  = (lo + 2 * w < n) ? lo + 2 * w : n;                                    \
        NAME##_merge(sk, si, dk, di, lo, mid, hi);                                               \
      }                                                                                          \
      T* xk = sk; sk = dk; dk = xk;                                                              \
      int64_t* xi = si; si = di; di = xi;                                                        \
    }                                                                                            \
    if (sk != k) {                                                                               \
      memcpy(k, sk, n * sizeof(T));                                                              \
      if (ix) memcpy(ix, si, n * sizeof(int64_t));                                               \
    }                                                                                            \
  }                                                                                              \
  static void NAME##_segment(T* k, int64_t* ix, T* tk, int64_t* ti, size_t n, int threads)       \
  {                                                                                              \
    if (threads <= 1 || n < 65536) {                                                             \
      NAME##_block(k, ix, tk, ti, n);                                                            \
      return;                                                                                    \
    }                                                                                            \
    int blocks = 1;                                                                              \
    while (blocks * 2 <= threads) blocks *= 2;                                                   \
    const size_t bs = (n + blocks - 1) / blocks;                                                 \
    _Pragma("omp parallel for num_threads(threads) schedule(static)")                            \
    for (int b = 0; b < blocks; ++b) {                                                           \
      const size_t lo = (size_t)b * bs;                                                          \
      if (lo < n) {                                                                              \
        const size_t len = (n - lo < bs) ? n - lo : bs;                                          \
        NAME##_block(k + lo, ix ? ix + lo : NULL, tk + lo, ti ? ti + lo : NULL, len);            \
      }                                                                                          \
    }                                                                                            \
    T* sk       = k;                                                                             \
    int64_t* si = ix;                                                                            \
    T* dk       = tk;                                                                            \
    int64_t* di = ti;                                                                            \
    for (size_t w = bs; w < n; w *= 2) {                                                         \
      const long pairs = (long)((n + 2 * w - 1) / (2 * w));                                      \
      _Pragma("omp parallel for num_threads(threads) schedule(static)")                          \
      for (long p = 0; p < pairs; ++p) {                                                         \
        const size_t lo  = (size_t)p * 2 * w;                                                    \
        const size_t mid = (lo + w < n) ? lo + w : n;                                            \
        const size_t hi  = (lo + 2 * w < n) ? lo + 2 * w : n;                                    \
        NAME##_merge(sk, si, dk, di, lo, mid, hi);                                               \
      }                                                                                          \
      T* xk = sk; sk = dk; dk = xk;                                                              \
      int64_t* xi = si; si = di; di = xi;                                                        \
    }                                                                                            \
    if (sk != k) {                                                                               \
      memcpy(k, sk, n * sizeof(T));                                                              \
      if (ix) memcpy(ix, si, n * sizeof(int64_t));                                               \
    }                                                                                            \
  }                                                                                              \
  /* thrust_local_sort_inplace: serial loop over the segments */                                 \
  static int NAME##_local_sort_inplace(T* values, int64_t* indices, size_t volume, size_t seg,   \
                                       int threads)                                              \
  {                                                                                              \
    T* tk       = (T*)malloc((seg ? seg : 1) * sizeof(T));                                       \
    int64_t* ti = indices ? (int64_t*)malloc((seg ? seg : 1) * sizeof(int64_t)) : NULL;          \
    if (!tk || (indices && !ti)) {                                                               \
      free(tk);                                                                                  \
      free(ti);                                                                                  \
      return -1;                                                                                 \
    }                                                                                            \
    for (size_t start = 0; start < volume; start += seg) {                                       \
      NAME##_segment(values + start, indices ? indices + start : NULL, tk, ti, seg, threads);    \
    }                                                                                            \
    free(tk);                                                                                    \
    free(ti);                                                                                    \
    return 0;                                                                                    \
  }

DEFINE_SORT(s_u8, uint8_t, LESS_INT)
DEFINE_SORT(s_i8, int8_t, LESS_INT)
DEFINE_SORT(s_u16, uint16_t, LESS_INT)
DEFINE_SORT(s_i16, int16_t, LESS_INT)
DEFINE_SORT(s_u32, uint32_t, LESS_INT)
DEFINE_SORT(s_i32, int32_t, LESS_INT)
DEFINE_SORT(s_u64, uint64_t, LESS_INT)
DEFINE_SORT(s_i64, int64_t, LESS_INT)
DEFINE_SORT(s_f16, uint16_t, less_f16)
DEFINE_SORT(s_f32, float, less_f32)
DEFINE_SORT(s_f64, double, less_f64)
DEFINE_SORT(s_c64, c64_t, less_c64)
DEFINE_SORT(s_c128, c128_t, less_c128)

static size_t elem_size(int dtype)
{
  switch (dtype) {
    case T_BOOL: case T_I8: case T_U8: return 1;
    case T_I16: case T_U16: case T_F16: return 2;
    case T_I32: case T_U32: case T_F32: return 4;
    case T_I64: case T_U64: case T_F64: case T_C64: return 8;
    case T_C128: return 16;
    default: return 0;
  }
}

/*
 * SortImplBodyCpu, single-processor branch (need_distributed_sort == false).
 *
 *   input     dense row-major, volume elements, rows of `seg`
 *   values    receives the sorted values (for argsort this is the reference's key copy)
 *   indices   NULL for sort; else receives i % seg + offset, permuted with the keys
 *   threads   1 = thrust::host (CPU variant), >1 = thrust::omp::par (OMP variant)
 *
 * Returns 0, -1 out of memory, -2 bad arguments.
 */
int cpn_oracle_local_sort(int dtype, const void* input, void* values, int64_t* indices, uint64_t volume,
                          uint64_t seg, int64_t offset, int stable, int threads)
{
  (void)stable;
  const size_t es = elem_size(dtype);
  if (es == 0 || (volume != 0 && (seg == 0 || volume % seg != 0)) || (volume != 0 && (!input || !values))) {
    return -2;
  }
  if (volume == 0) {
    return 0;
  }
  if (indices) { /* sort_cpu.inl:990-1002 */
    for (uint64_t i = 0; i < volume; ++i) {
      indices[i] = (int64_t)(i % seg) + offset;
    }
  }
  if (input != values) { /* sort_cpu.inl:1022-1025 */
    memcpy(values, input, volume * es);
  }
  switch (dtype) {
    case T_BOOL:
    case T_U8: return s_u8_local_sort_inplace((uint8_t*)values, indices, volume, seg, threads);
    case T_I8: return s_i8_local_sort_inplace((int8_t*)values, indices, volume, seg, threads);
    case T_U16: return s_u16_local_sort_inplace((uint16_t*)values, indices, volume, seg, threads);
    case T_I16: return s_i16_local_sort_inplace((int16_t*)values, indices, volume, seg, threads);
    case T_U32: return s_u32_local_sort_inplace((uint32_t*)values, indices, volume, seg, threads);
    case T_I32: return s_i32_local_sort_inplace((int32_t*)values, indices, volume, seg, threads);
    case T_U64: return s_u64_local_sort_inplace((uint64_t*)values, indices, volume, seg, threads);
    case T_I64: return s_i64_local_sort_inplace((int64_t*)values, indices, volume, seg, threads);
    case T_F16: return s_f16_local_sort_inplace((uint16_t*)values, indices, volume, seg, threads);
    case T_F32: return s_f32_local_sort_inplace((float*)values, indices, volume, seg, threads);
    case T_F64: return s_f64_local_sort_inplace((double*)values, indices, volume, seg, threads);
    case T_C64: return s_c64_local_sort_inplace((c64_t*)values, indices, volume, seg, threads);
    case T_C128: return s_c128_local_sort_inplace((c128_t*)values, indices, volume, seg, threads);
    default: return -2;
  }
}

int cpn_oracle_max_threads(void)
{
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}
