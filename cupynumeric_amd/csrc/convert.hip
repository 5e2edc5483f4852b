// Element type conversion, the casts the sort path needs around its kernels:
//  * sort_complex returns complex64 for integers of at most 16 bits and complex128 for every
//    other real type (cupynumeric/_module/ssc_sorting.py:124-159, `result.astype(...)`);
//  * searchsorted brings the sorted array and the values to their common type first
//    (cupynumeric/_array/array.py:3743-3751, `astype(np.result_type(...))`).
// In the reference both are UNARY_OP tasks (src/cupynumeric/unary/convert.cu).  One kernel per
// (source, destination) pair; conversions follow C++ `static_cast` (float16 through float32),
// bool destinations are `x != 0`, complex -> real keeps the real part.
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "sort_driver.h"

namespace cpn {

struct BoolTag {};  // one byte, 0 or 1
template <typename F>
struct ComplexTag {};  // two F

// Element access by tag: load gives (re, im) in a carrier type that holds every value of the
// element type (the type itself, float for float16), store takes the same.
template <typename T>
struct Elem {
  using carrier = T;
  static constexpr bool is_complex = false;
  static __device__ __forceinline__ void load(const void* p, uint64_t i, carrier& re, carrier& im)
  {
    re = static_cast<const T*>(p)[i];
    im = carrier(0);
  }
  template <typename C>
  static __device__ __forceinline__ void store(void* p, uint64_t i, C re, C)
  {
    static_cast<T*>(p)[i] = static_cast<T>(re);
  }
};
// float16 from a wider value with ONE rounding to nearest even, as NumPy's casts do.  float32 goes
// through the hardware conversion.  float64 is first brought to float32 by truncation with the lost
// bits ORed into the last place ("round to odd"): float32 keeps 13 bits more than float16, so the
// second, proper rounding sees exactly what a direct one would.  64-bit integers go through float64
// (exact below 2^53, and everything from 65520 up is infinity in float16 either way).
__device__ __forceinline__ __half half_from(float v) { return __float2half(v); }
__device__ __forceinline__ __half half_from(double v)
{
  float f = __double2float_rz(v);
  if (v == v && static_cast<double>(f) != v) {  // inexact (not NaN): make the result odd
    uint32_t bits;
    __builtin_memcpy(&bits, &f, 4);
    bits |= 1u;
    __builtin_memcpy(&f, &bits, 4);
  }
  return __float2half(f);
}
__device__ __forceinline__ __half half_from(int64_t v) { return half_from(static_cast<double>(v)); }
__device__ __forceinline__ __half half_from(uint64_t v) { return half_from(static_cast<double>(v)); }
template <typename C>
__device__ __forceinline__ __half half_from(C v)  // narrower integers and bool bytes: exact in float32 below 65520
{
  return __float2half(static_cast<float>(v));
}

template <>
struct Elem<__half> {
  using carrier = float;
  static constexpr bool is_complex = false;
  static __device__ __forceinline__ void load(const void* p, uint64_t i, carrier& re, carrier& im)
  {
    re = __half2float(static_cast<const __half*>(p)[i]);
    im = 0.0f;
  }
  template <typename C>
  static __device__ __forceinline__ void store(void* p, uint64_t i, C re, C)
  {
    static_cast<__half*>(p)[i] = half_from(re);
  }
};
template <>
struct Elem<BoolTag> {
  using carrier = uint8_t;
  static constexpr bool is_complex = false;
  static __device__ __forceinline__ void load(const void* p, uint64_t i, carrier& re, carrier& im)
  {
    re = static_cast<const uint8_t*>(p)[i] != 0 ? 1 : 0;
    im = 0;
  }
  template <typename C>
  static __device__ __forceinline__ void store(void* p, uint64_t i, C re, C im)
  {
    static_cast<uint8_t*>(p)[i] = (re != C(0) || im != C(0)) ? 1 : 0;
  }
};
template <typename F>
struct Elem<ComplexTag<F>> {
  using carrier = F;
  static constexpr bool is_complex = true;
  static __device__ __forceinline__ void load(const void* p, uint64_t i, carrier& re, carrier& im)
  {
    re = static_cast<const F*>(p)[2 * i];
    im = static_cast<const F*>(p)[2 * i + 1];
  }
  template <typename C>
  static __device__ __forceinline__ void store(void* p, uint64_t i, C re, C im)
  {
    static_cast<F*>(p)[2 * i]     = static_cast<F>(re);
    static_cast<F*>(p)[2 * i + 1] = static_cast<F>(im);
  }
};

template <typename Src, typename Dst>
__global__ __launch_bounds__(256) void convert_kernel(const void* __restrict__ in, void* __restrict__ out, uint64_t n)
{
  const uint64_t stride = static_cast<uint64_t>(gridDim.x) * blockDim.x;
  for (uint64_t i = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n; i += stride) {
    typename Elem<Src>::carrier re, im;
    Elem<Src>::load(in, i, re, im);
    Elem<Dst>::store(out, i, re, im);
  }
}

template <typename Src, typename Dst>
static int launch_convert(const void* in, void* out, uint64_t n, hipStream_t stream)
{
  uint64_t grid = (n + 255) / 256;
  if (grid > 65536) {
    grid = 65536;
  }
  ProfileScope prof("convert", stream);
  hipLaunchKernelGGL((convert_kernel<Src, Dst>), dim3(static_cast<uint32_t>(grid)), dim3(256), 0, stream, in, out, n);
  CPN_HIP_TRY(hipGetLastError());
  return CPN_OK;
}

template <typename Src>
static int convert_from(int dst_dtype, const void* in, void* out, uint64_t n, hipStream_t stream)
{
  switch (dst_dtype) {
    case CPN_BOOL: return launch_convert<Src, BoolTag>(in, out, n, stream);
    case CPN_INT8: return launch_convert<Src, int8_t>(in, out, n, stream);
    case CPN_INT16: return launch_convert<Src, int16_t>(in, out, n, stream);
    case CPN_INT32: return launch_convert<Src, int32_t>(in, out, n, stream);
    case CPN_INT64: return launch_convert<Src, int64_t>(in, out, n, stream);
    case CPN_UINT8: return launch_convert<Src, uint8_t>(in, out, n, stream);
    case CPN_UINT16: return launch_convert<Src, uint16_t>(in, out, n, stream);
    case CPN_UINT32: return launch_convert<Src, uint32_t>(in, out, n, stream);
    case CPN_UINT64: return launch_convert<Src, uint64_t>(in, out, n, stream);
    case CPN_FLOAT16: return launch_convert<Src, __half>(in, out, n, stream);
    case CPN_FLOAT32: return launch_convert<Src, float>(in, out, n, stream);
    case CPN_FLOAT64: return launch_convert<Src, double>(in, out, n, stream);
    case CPN_COMPLEX64: return launch_convert<Src, ComplexTag<float>>(in, out, n, stream);
    case CPN_COMPLEX128: return launch_convert<Src, ComplexTag<double>>(in, out, n, stream);
    default: return CPN_ERR_DTYPE;
  }
}

static int convert_dispatch(int src_dtype, const void* in, int dst_dtype, void* out, uint64_t n, hipStream_t stream)
{
  switch (src_dtype) {
    case CPN_BOOL: return convert_from<BoolTag>(dst_dtype, in, out, n, stream);
    case CPN_INT8: return convert_from<int8_t>(dst_dtype, in, out, n, stream);
    case CPN_INT16: return convert_from<int16_t>(dst_dtype, in, out, n, stream);
    case CPN_INT32: return convert_from<int32_t>(dst_dtype, in, out, n, stream);
    case CPN_INT64: return convert_from<int64_t>(dst_dtype, in, out, n, stream);
    case CPN_UINT8: return convert_from<uint8_t>(dst_dtype, in, out, n, stream);
    case CPN_UINT16: return convert_from<uint16_t>(dst_dtype, in, out, n, stream);
    case CPN_UINT32: return convert_from<uint32_t>(dst_dtype, in, out, n, stream);
    case CPN_UINT64: return convert_from<uint64_t>(dst_dtype, in, out, n, stream);
    case CPN_FLOAT16: return convert_from<__half>(dst_dtype, in, out, n, stream);
    case CPN_FLOAT32: return convert_from<float>(dst_dtype, in, out, n, stream);
    case CPN_FLOAT64: return convert_from<double>(dst_dtype, in, out, n, stream);
    case CPN_COMPLEX64: return convert_from<ComplexTag<float>>(dst_dtype, in, out, n, stream);
    case CPN_COMPLEX128: return convert_from<ComplexTag<double>>(dst_dtype, in, out, n, stream);
    default: return CPN_ERR_DTYPE;
  }
}

}  // namespace cpn

extern "C" int cpn_astype(int src_dtype, const void* in, int dst_dtype, void* out, uint64_t volume, void* stream)
{
  if (src_dtype < CPN_BOOL || src_dtype > CPN_COMPLEX128 || dst_dtype < CPN_BOOL || dst_dtype > CPN_COMPLEX128) {
    return CPN_ERR_DTYPE;
  }
  if (volume == 0) {
    return CPN_OK;
  }
  if (in == nullptr || out == nullptr) {
    return CPN_ERR_NULL;
  }
  return cpn::convert_dispatch(src_dtype, in, dst_dtype, out, volume, static_cast<hipStream_t>(stream));
}

extern "C" int cpn_real_to_complex(int src_dtype, const void* in, int dst_dtype, void* out, uint64_t volume, void* stream)
{
  if (dst_dtype != CPN_COMPLEX64 && dst_dtype != CPN_COMPLEX128) {
    return CPN_ERR_DTYPE;
  }
  if (src_dtype < CPN_BOOL || src_dtype > CPN_FLOAT64) {
    return CPN_ERR_DTYPE;
  }
  return cpn_astype(src_dtype, in, dst_dtype, out, volume, stream);
}
