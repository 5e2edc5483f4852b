// Quantiles of rows that are already sorted: for every requested quantile, the element at a
// precomputed position of the sort axis, or the weighted sum of two neighbouring elements.
//
// Replaces the tail of _quantile_impl (cupynumeric/_module/stats_order.py:249-337): per quantile,
//   arr.take(left, axis)                                         (methods that do not interpolate)
//   (1.0 - gamma) * arr.take(left, axis) + gamma * arr.take(right, axis), stored as float64
// which the reference issues as take / multiply / add / assignment tasks per quantile; here one
// launch evaluates all quantiles.  The arithmetic is the reference's, operation for operation and
// in the type its expressions have: the element type for float16 / float32 / float64 arrays (a
// Python float times such an array keeps the array's type), float64 for integer and bool arrays;
// two products, one sum, no fused multiply-add.
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "sort_driver.h"

namespace cpn {

// The reference's expression in the arithmetic of `T`'s array type; the result as float64.
template <typename T>
struct Lerp {  // integers and bool bytes: promoted to float64
  static __device__ __forceinline__ double eval(T l, T r, double gamma)
  {
#pragma clang fp contract(off)  // two rounded products and a rounded sum, never a fused multiply-add
    const double a = (1.0 - gamma) * static_cast<double>(l);
    const double b = gamma * static_cast<double>(r);
    return a + b;
  }
};
template <>
struct Lerp<double> {
  static __device__ __forceinline__ double eval(double l, double r, double gamma)
  {
#pragma clang fp contract(off)
    const double a = (1.0 - gamma) * l;
    const double b = gamma * r;
    return a + b;
  }
};
template <>
struct Lerp<float> {
  static __device__ __forceinline__ double eval(float l, float r, double gamma)
  {
#pragma clang fp contract(off)
    const float m1 = static_cast<float>(1.0 - gamma), g = static_cast<float>(gamma);  // the scalars take the array's type
    const float a = m1 * l;
    const float b = g * r;
    return static_cast<double>(a + b);
  }
};
// float16 arithmetic as NumPy does it: operands widened to float32, one operation, rounded back
// (a product of two float16 numbers is exact in float32).  The scalars are rounded from float64 once.
__device__ __forceinline__ float half_round(float v) { return __half2float(__float2half(v)); }
__device__ __forceinline__ float half_of_double(double v)
{
  float f = __double2float_rz(v);
  if (v == v && static_cast<double>(f) != v) {  // inexact: round to odd first, then the proper rounding is exact
    uint32_t bits;
    __builtin_memcpy(&bits, &f, 4);
    bits |= 1u;
    __builtin_memcpy(&f, &bits, 4);
  }
  return half_round(f);
}
template <>
struct Lerp<__half> {
  static __device__ __forceinline__ double eval(__half l, __half r, double gamma)
  {
#pragma clang fp contract(off)
    const float m1 = half_of_double(1.0 - gamma), g = half_of_double(gamma);
    const float a  = half_round(m1 * __half2float(l));
    const float b  = half_round(g * __half2float(r));
    return static_cast<double>(half_round(a + b));
  }
};

// sorted: [outer][n][inner]; out: [num_q][outer][inner].  One thread per output element.
template <typename T, bool INTERPOLATE>
__global__ __launch_bounds__(256) void quantile_kernel(const T* __restrict__ sorted,
                                                       uint64_t outer,
                                                       uint64_t n,
                                                       uint64_t inner,
                                                       uint64_t num_q,
                                                       const int64_t* __restrict__ left,
                                                       const int64_t* __restrict__ right,
                                                       const double* __restrict__ gamma,
                                                       void* __restrict__ out)
{
  const uint64_t per_q  = outer * inner;
  const uint64_t total  = num_q * per_q;
  const uint64_t stride = static_cast<uint64_t>(gridDim.x) * blockDim.x;
  for (uint64_t e = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x; e < total; e += stride) {
    const uint64_t q    = e / per_q;
    const uint64_t rest = e - q * per_q;
    const uint64_t o    = rest / inner;
    const uint64_t i    = rest - o * inner;
    const T* column     = sorted + o * n * inner + i;
    const T l           = column[static_cast<uint64_t>(left[q]) * inner];
    if constexpr (INTERPOLATE) {
      const T r                    = column[static_cast<uint64_t>(right[q]) * inner];
      static_cast<double*>(out)[e] = Lerp<T>::eval(l, r, gamma[q]);
    } else {
      static_cast<T*>(out)[e] = l;
    }
  }
}

template <typename T>
static int launch_quantile(const void* sorted, uint64_t outer, uint64_t n, uint64_t inner, uint64_t num_q,
                           const int64_t* left, const int64_t* right, const double* gamma, int interpolate, void* out,
                           hipStream_t stream)
{
  const uint64_t total = num_q * outer * inner;
  uint64_t grid        = (total + 255) / 256;
  if (grid > 65536) {
    grid = 65536;
  }
  ProfileScope prof("quantile", stream);
  if (interpolate) {
    hipLaunchKernelGGL((quantile_kernel<T, true>), dim3(static_cast<uint32_t>(grid)), dim3(256), 0, stream,
                       static_cast<const T*>(sorted), outer, n, inner, num_q, left, right, gamma, out);
  } else {
    hipLaunchKernelGGL((quantile_kernel<T, false>), dim3(static_cast<uint32_t>(grid)), dim3(256), 0, stream,
                       static_cast<const T*>(sorted), outer, n, inner, num_q, left, right, gamma, out);
  }
  CPN_HIP_TRY(hipGetLastError());
  return CPN_OK;
}

// ---- the variants that ignore NaNs ---------------------------------------------------------------------
// NaN test and the two constants the reference's view of a slice needs, per float type.
template <typename T> struct FloatBits;
template <> struct FloatBits<__half> {
  using U = uint16_t;
  static constexpr U INF = 0x7C00u, MAXV = 0x7BFFu, ABS = 0x7FFFu, QNAN = 0x7E00u;
};
template <> struct FloatBits<float> {
  using U = uint32_t;
  static constexpr U INF = 0x7F800000u, MAXV = 0x7F7FFFFFu, ABS = 0x7FFFFFFFu, QNAN = 0x7FC00000u;
};
template <> struct FloatBits<double> {
  using U = uint64_t;
  static constexpr U INF = 0x7FF0000000000000ull, MAXV = 0x7FEFFFFFFFFFFFFFull, ABS = 0x7FFFFFFFFFFFFFFFull,
                     QNAN = 0x7FF8000000000000ull;
};
template <typename T>
__device__ __forceinline__ typename FloatBits<T>::U bits_of(T v)
{
  typename FloatBits<T>::U b;
  __builtin_memcpy(&b, &v, sizeof(T));
  return b;
}
template <typename T>
__device__ __forceinline__ T from_bits(typename FloatBits<T>::U b)
{
  T v;
  __builtin_memcpy(&v, &b, sizeof(T));
  return v;
}
template <typename T>
__device__ __forceinline__ bool is_nan_bits(T v)
{
  return (bits_of(v) & FloatBits<T>::ABS) > FloatBits<T>::INF;
}

// First position in [0, hi) of a column (stride `inner`) whose element satisfies `pred`, for a
// predicate that is false on a prefix and true on the rest.
template <typename T, typename Pred>
__device__ __forceinline__ uint64_t first_where(const T* column, uint64_t inner, uint64_t hi, Pred pred)
{
  uint64_t lo = 0;
  while (lo < hi) {
    const uint64_t mid = lo + (hi - lo) / 2;
    if (pred(column[mid * inner])) {
      hi = mid;
    } else {
      lo = mid + 1;
    }
  }
  return lo;
}

template <typename T>
__global__ __launch_bounds__(256) void count_not_nan_kernel(const T* __restrict__ sorted, uint64_t outer, uint64_t n,
                                                            uint64_t inner, int64_t* __restrict__ counts)
{
  const uint64_t total  = outer * inner;
  const uint64_t stride = static_cast<uint64_t>(gridDim.x) * blockDim.x;
  for (uint64_t e = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x; e < total; e += stride) {
    const uint64_t o = e / inner, i = e - o * inner;
    const T* column  = sorted + o * n * inner + i;
    counts[e]        = static_cast<int64_t>(first_where(column, inner, n, [](T v) { return is_nan_bits(v); }));
  }
}

// The reference's expression on arrays of the element type (stats_order.py:748-757): gamma stored in
// an array of that type, `1 - gammas`, two products and a sum, each rounded in that type.
template <typename T>
struct NanLerp {
  static __device__ __forceinline__ T eval(T l, T r, double gamma)
  {
#pragma clang fp contract(off)
    const T g  = static_cast<T>(gamma);
    const T m1 = static_cast<T>(1) - g;
    const T a  = m1 * l;
    const T b  = g * r;
    return a + b;
  }
};
template <>
struct NanLerp<__half> {
  static __device__ __forceinline__ __half eval(__half l, __half r, double gamma)
  {
#pragma clang fp contract(off)
    const float g  = half_of_double(gamma);
    const float m1 = half_round(1.0f - g);
    const float a  = half_round(m1 * __half2float(l));
    const float b  = half_round(g * __half2float(r));
    return __float2half(half_round(a + b));
  }
};
template <typename T> __device__ __forceinline__ double widen(T v) { return static_cast<double>(v); }
template <> __device__ __forceinline__ double widen<__half>(__half v) { return static_cast<double>(__half2float(v)); }

// sorted: [outer][n][inner]; counts: [outer][inner]; left, right, gamma, out: [num_q][outer][inner].
template <typename T, bool INTERPOLATE, bool KEEP>
__global__ __launch_bounds__(256) void nanquantile_kernel(const T* __restrict__ sorted, uint64_t outer, uint64_t n,
                                                          uint64_t inner, uint64_t num_q,
                                                          const int64_t* __restrict__ counts,
                                                          const int64_t* __restrict__ left,
                                                          const int64_t* __restrict__ right,
                                                          const double* __restrict__ gamma, void* __restrict__ out)
{
  using FB              = FloatBits<T>;
  const uint64_t per_q  = outer * inner;
  const uint64_t total  = num_q * per_q;
  const uint64_t stride = static_cast<uint64_t>(gridDim.x) * blockDim.x;
  for (uint64_t e = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x; e < total; e += stride) {
    const uint64_t q    = e / per_q;
    const uint64_t rest = e - q * per_q;
    const uint64_t o    = rest / inner;
    const uint64_t i    = rest - o * inner;
    const T* column     = sorted + o * n * inner + i;
    const uint64_t kept = static_cast<uint64_t>(counts[rest]);
    T value             = from_bits<T>(FB::QNAN);
    if (kept != 0) {
      // the slice as the reference sorts it: finite elements, then its NaNs as the largest finite value, then +inf
      const uint64_t nans   = n - kept;
      const uint64_t finite = nans == 0 ? kept : first_where(column, inner, kept, [](T v) { return bits_of(v) == FB::INF; });
      auto at = [&](uint64_t p) -> T {
        if (p < finite) {
          return column[p * inner];
        }
        return from_bits<T>(p < finite + nans ? FB::MAXV : FB::INF);
      };
      const T l = at(static_cast<uint64_t>(left[e]));
      if constexpr (INTERPOLATE) {
        value = NanLerp<T>::eval(l, at(static_cast<uint64_t>(right[e])), gamma[e]);
      } else {
        value = l;
      }
    }
    if constexpr (KEEP) {
      static_cast<T*>(out)[e] = value;
    } else {
      static_cast<double*>(out)[e] = widen(value);
    }
  }
}

template <typename T>
static int launch_nanquantile(const void* sorted, uint64_t outer, uint64_t n, uint64_t inner, uint64_t num_q,
                              const int64_t* counts, const int64_t* left, const int64_t* right, const double* gamma,
                              int interpolate, int keep, void* out, hipStream_t stream)
{
  const uint64_t total = num_q * outer * inner;
  uint64_t grid        = (total + 255) / 256;
  if (grid > 65536) {
    grid = 65536;
  }
  const dim3 g(static_cast<uint32_t>(grid)), b(256);
  const T* in = static_cast<const T*>(sorted);
  ProfileScope prof("nanquantile", stream);
  if (interpolate && keep) {
    hipLaunchKernelGGL((nanquantile_kernel<T, true, true>), g, b, 0, stream, in, outer, n, inner, num_q, counts, left, right, gamma, out);
  } else if (interpolate) {
    hipLaunchKernelGGL((nanquantile_kernel<T, true, false>), g, b, 0, stream, in, outer, n, inner, num_q, counts, left, right, gamma, out);
  } else if (keep) {
    hipLaunchKernelGGL((nanquantile_kernel<T, false, true>), g, b, 0, stream, in, outer, n, inner, num_q, counts, left, right, gamma, out);
  } else {
    hipLaunchKernelGGL((nanquantile_kernel<T, false, false>), g, b, 0, stream, in, outer, n, inner, num_q, counts, left, right, gamma, out);
  }
  CPN_HIP_TRY(hipGetLastError());
  return CPN_OK;
}

template <typename T>
static int launch_count_not_nan(const void* sorted, uint64_t outer, uint64_t n, uint64_t inner, int64_t* counts,
                                hipStream_t stream)
{
  const uint64_t total = outer * inner;
  uint64_t grid        = (total + 255) / 256;
  if (grid > 65536) {
    grid = 65536;
  }
  ProfileScope prof("count_not_nan", stream);
  hipLaunchKernelGGL((count_not_nan_kernel<T>), dim3(static_cast<uint32_t>(grid)), dim3(256), 0, stream,
                     static_cast<const T*>(sorted), outer, n, inner, counts);
  CPN_HIP_TRY(hipGetLastError());
  return CPN_OK;
}

}  // namespace cpn

extern "C" int cpn_count_not_nan_sorted(int dtype, const void* sorted, uint64_t outer, uint64_t n, uint64_t inner,
                                        int64_t* counts, void* stream)
{
  if (dtype != CPN_FLOAT16 && dtype != CPN_FLOAT32 && dtype != CPN_FLOAT64) {
    return CPN_ERR_DTYPE;
  }
  if (outer == 0 || inner == 0) {
    return CPN_OK;
  }
  if (counts == nullptr || (sorted == nullptr && n != 0)) {
    return CPN_ERR_NULL;
  }
  const uintptr_t elem = dtype == CPN_FLOAT16 ? 2u : (dtype == CPN_FLOAT32 ? 4u : 8u);
  if ((reinterpret_cast<uintptr_t>(sorted) & (elem - 1)) != 0 || (reinterpret_cast<uintptr_t>(counts) & 7u) != 0) {
    return CPN_ERR_ALIGN;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (dtype) {
    case CPN_FLOAT16: return cpn::launch_count_not_nan<__half>(sorted, outer, n, inner, counts, s);
    case CPN_FLOAT32: return cpn::launch_count_not_nan<float>(sorted, outer, n, inner, counts, s);
    default: return cpn::launch_count_not_nan<double>(sorted, outer, n, inner, counts, s);
  }
}

extern "C" int cpn_nanquantile_sorted(int dtype, const void* sorted, uint64_t outer, uint64_t n, uint64_t inner,
                                      uint64_t num_q, const int64_t* counts, const int64_t* left, const int64_t* right,
                                      const double* gamma, int interpolate, int keep_dtype, void* out, void* stream)
{
  if (dtype != CPN_FLOAT16 && dtype != CPN_FLOAT32 && dtype != CPN_FLOAT64) {
    return CPN_ERR_DTYPE;
  }
  if (num_q == 0 || outer == 0 || inner == 0) {
    return CPN_OK;
  }
  if (counts == nullptr || left == nullptr || out == nullptr || (sorted == nullptr && n != 0) ||
      (interpolate != 0 && (right == nullptr || gamma == nullptr))) {
    return CPN_ERR_NULL;
  }
  const uintptr_t elem     = dtype == CPN_FLOAT16 ? 2u : (dtype == CPN_FLOAT32 ? 4u : 8u);
  const uintptr_t out_mask = keep_dtype != 0 ? elem - 1 : 7u;
  if ((reinterpret_cast<uintptr_t>(sorted) & (elem - 1)) != 0 || (reinterpret_cast<uintptr_t>(out) & out_mask) != 0 ||
      (reinterpret_cast<uintptr_t>(counts) & 7u) != 0 || (reinterpret_cast<uintptr_t>(left) & 7u) != 0 ||
      (reinterpret_cast<uintptr_t>(right) & 7u) != 0 || (reinterpret_cast<uintptr_t>(gamma) & 7u) != 0) {
    return CPN_ERR_ALIGN;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (dtype) {
    case CPN_FLOAT16:
      return cpn::launch_nanquantile<__half>(sorted, outer, n, inner, num_q, counts, left, right, gamma, interpolate, keep_dtype, out, s);
    case CPN_FLOAT32:
      return cpn::launch_nanquantile<float>(sorted, outer, n, inner, num_q, counts, left, right, gamma, interpolate, keep_dtype, out, s);
    default:
      return cpn::launch_nanquantile<double>(sorted, outer, n, inner, num_q, counts, left, right, gamma, interpolate, keep_dtype, out, s);
  }
}

extern "C" int cpn_quantile_sorted(int dtype, const void* sorted, uint64_t outer, uint64_t n, uint64_t inner,
                                   uint64_t num_q, const int64_t* left, const int64_t* right, const double* gamma,
                                   int interpolate, void* out, void* stream)
{
  const cpn::KeyKind k = cpn::key_kind(dtype);
  if (k.bytes == 0 || k.codec == cpn::CODEC_COMPLEX) {
    return CPN_ERR_DTYPE;
  }
  if (num_q == 0 || outer == 0 || inner == 0) {
    return CPN_OK;
  }
  if (n == 0) {
    return CPN_ERR_SHAPE;  // no element to take
  }
  if (sorted == nullptr || left == nullptr || out == nullptr || (interpolate != 0 && (right == nullptr || gamma == nullptr))) {
    return CPN_ERR_NULL;
  }
  const uintptr_t out_mask = interpolate != 0 ? 7u : static_cast<uintptr_t>(k.bytes - 1);
  if ((reinterpret_cast<uintptr_t>(sorted) & static_cast<uintptr_t>(k.bytes - 1)) != 0 ||
      (reinterpret_cast<uintptr_t>(out) & out_mask) != 0 || (reinterpret_cast<uintptr_t>(left) & 7u) != 0 ||
      (reinterpret_cast<uintptr_t>(right) & 7u) != 0 || (reinterpret_cast<uintptr_t>(gamma) & 7u) != 0) {
    return CPN_ERR_ALIGN;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (dtype) {
    case CPN_BOOL: return cpn::launch_quantile<uint8_t>(sorted, outer, n, inner, num_q, left, right, gamma, interpolate, out, s);
    case CPN_INT8: return cpn::launch_quantile<int8_t>(sorted, outer, n, inner, num_q, left, right, gamma, interpolate, out, s);
    case CPN_INT16: return cpn::launch_quantile<int16_t>(sorted, outer, n, inner, num_q, left, right, gamma, interpolate, out, s);
    case CPN_INT32: return cpn::launch_quantile<int32_t>(sorted, outer, n, inner, num_q, left, right, gamma, interpolate, out, s);
    case CPN_INT64: return cpn::launch_quantile<int64_t>(sorted, outer, n, inner, num_q, left, right, gamma, interpolate, out, s);
    case CPN_UINT8: return cpn::launch_quantile<uint8_t>(sorted, outer, n, inner, num_q, left, right, gamma, interpolate, out, s);
    case CPN_UINT16: return cpn::launch_quantile<uint16_t>(sorted, outer, n, inner, num_q, left, right, gamma, interpolate, out, s);
    case CPN_UINT32: return cpn::launch_quantile<uint32_t>(sorted, outer, n, inner, num_q, left, right, gamma, interpolate, out, s);
    case CPN_UINT64: return cpn::launch_quantile<uint64_t>(sorted, outer, n, inner, num_q, left, right, gamma, interpolate, out, s);
    case CPN_FLOAT16: return cpn::launch_quantile<__half>(sorted, outer, n, inner, num_q, left, right, gamma, interpolate, out, s);
    case CPN_FLOAT32: return cpn::launch_quantile<float>(sorted, outer, n, inner, num_q, left, right, gamma, interpolate, out, s);
    case CPN_FLOAT64: return cpn::launch_quantile<double>(sorted, outer, n, inner, num_q, left, right, gamma, interpolate, out, s);
    default: return CPN_ERR_DTYPE;
  }
}
