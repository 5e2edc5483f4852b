// Real -> complex element conversion, the one cast the sort path needs: sort_complex returns
// complex64 for integers of at most 16 bits and complex128 for every other real type
// (cupynumeric/_module/ssc_sorting.py:124-159, where it is `result.astype(...)`, a UNARY_OP
// task in the reference).
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "sort_driver.h"

namespace cpn {

template <typename Src, typename Part>
__global__ __launch_bounds__(256) void to_complex_kernel(const Src* __restrict__ in, Part* __restrict__ out, uint64_t n)
{
  const uint64_t stride = static_cast<uint64_t>(gridDim.x) * blockDim.x;
  for (uint64_t i = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n; i += stride) {
    Part re;
    if constexpr (sizeof(Src) == 2 && !std::is_integral<Src>::value) {
      re = static_cast<Part>(__half2float(in[i]));
    } else {
      re = static_cast<Part>(in[i]);
    }
    out[2 * i]     = re;
    out[2 * i + 1] = static_cast<Part>(0);
  }
}

template <typename Src, typename Part>
static int launch_to_complex(const void* in, void* out, uint64_t n, hipStream_t stream)
{
  uint64_t grid = (n + 255) / 256;
  if (grid > 65536) {
    grid = 65536;
  }
  ProfileScope prof("to_complex", stream);
  hipLaunchKernelGGL((to_complex_kernel<Src, Part>), dim3(static_cast<uint32_t>(grid)), dim3(256), 0, stream,
                     static_cast<const Src*>(in), static_cast<Part*>(out), n);
  CPN_HIP_TRY(hipGetLastError());
  return CPN_OK;
}

template <typename Part>
static int to_complex_dispatch(int src_dtype, const void* in, void* out, uint64_t n, hipStream_t stream)
{
  switch (src_dtype) {
    case CPN_BOOL: return launch_to_complex<uint8_t, Part>(in, out, n, stream);  // bytes are 0 / 1
    case CPN_INT8: return launch_to_complex<int8_t, Part>(in, out, n, stream);
    case CPN_INT16: return launch_to_complex<int16_t, Part>(in, out, n, stream);
    case CPN_INT32: return launch_to_complex<int32_t, Part>(in, out, n, stream);
    case CPN_INT64: return launch_to_complex<int64_t, Part>(in, out, n, stream);
    case CPN_UINT8: return launch_to_complex<uint8_t, Part>(in, out, n, stream);
    case CPN_UINT16: return launch_to_complex<uint16_t, Part>(in, out, n, stream);
    case CPN_UINT32: return launch_to_complex<uint32_t, Part>(in, out, n, stream);
    case CPN_UINT64: return launch_to_complex<uint64_t, Part>(in, out, n, stream);
    case CPN_FLOAT16: return launch_to_complex<__half, Part>(in, out, n, stream);
    case CPN_FLOAT32: return launch_to_complex<float, Part>(in, out, n, stream);
    case CPN_FLOAT64: return launch_to_complex<double, Part>(in, out, n, stream);
    default: return CPN_ERR_DTYPE;
  }
}

}  // namespace cpn

extern "C" int cpn_real_to_complex(int src_dtype, const void* in, int dst_dtype, void* out, uint64_t volume, void* stream)
{
  if (dst_dtype != CPN_COMPLEX64 && dst_dtype != CPN_COMPLEX128) {
    return CPN_ERR_DTYPE;
  }
  if (src_dtype < CPN_BOOL || src_dtype > CPN_FLOAT64) {
    return CPN_ERR_DTYPE;
  }
  if (volume == 0) {
    return CPN_OK;
  }
  if (in == nullptr || out == nullptr) {
    return CPN_ERR_NULL;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  return dst_dtype == CPN_COMPLEX64 ? cpn::to_complex_dispatch<float>(src_dtype, in, out, volume, s)
                                    : cpn::to_complex_dispatch<double>(src_dtype, in, out, volume, s);
}
