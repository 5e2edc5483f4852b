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

}  // namespace cpn

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
