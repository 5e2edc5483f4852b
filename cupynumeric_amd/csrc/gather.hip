// Gather along the last axis of dense rows: out[r][j] = src[r][idx[r][j]].
//
// This is what lexsort needs from take_along_axis (cupynumeric/_module/ssc_sorting.py:430-442:
// every further key is reordered by the current indices, and the indices by the new order;
// take_along_axis itself is cupynumeric/_module/indexing.py:648-760).  Axes other than the
// last are brought there by the transpose of swapaxes.hip first.
//
// One thread per output element group: index reads and output writes are contiguous along a
// wavefront; the source reads are the scattered part and stay inside one row.  Indices may be
// negative (counted from the end of the row, as in NumPy); an index outside [-n, n) sets a
// flag and writes nothing, the host turns the flag into IndexError.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "sort_driver.h"

namespace cpn {

template <typename T>
__global__ __launch_bounds__(256) void take_last_axis_kernel(const T* __restrict__ src,
                                                              const int64_t* __restrict__ idx,
                                                              T* __restrict__ out,
                                                              uint64_t total,
                                                              uint64_t src_seg,
                                                              uint64_t idx_seg,
                                                              uint32_t* oob_flag)
{
  const uint64_t stride = static_cast<uint64_t>(gridDim.x) * blockDim.x;
  bool bad              = false;
  for (uint64_t o = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x; o < total; o += stride) {
    const uint64_t row = o / idx_seg;
    int64_t k          = idx[o];
    if (k < 0) {
      k += static_cast<int64_t>(src_seg);
    }
    if (k < 0 || static_cast<uint64_t>(k) >= src_seg) {
      bad = true;
    } else {
      out[o] = src[row * src_seg + static_cast<uint64_t>(k)];
    }
  }
  if (bad && oob_flag != nullptr) {
    __hip_atomic_store(oob_flag, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}

template <typename T>
static int launch_take(const void* src, const int64_t* idx, void* out, uint64_t rows, uint64_t src_seg,
                       uint64_t idx_seg, uint32_t* oob_flag, hipStream_t stream)
{
  const uint64_t total = rows * idx_seg;
  uint64_t grid        = (total + 255) / 256;
  if (grid > (1u << 20)) {
    grid = 1u << 20;
  }
  ProfileScope prof("take_last_axis", stream);
  hipLaunchKernelGGL((take_last_axis_kernel<T>), dim3(static_cast<uint32_t>(grid)), dim3(256), 0, stream,
                     static_cast<const T*>(src), idx, static_cast<T*>(out), total, src_seg, idx_seg, oob_flag);
  CPN_HIP_TRY(hipGetLastError());
  return CPN_OK;
}

}  // namespace cpn

extern "C" int cpn_take_along_last_axis(int elem_bytes, const void* src, const int64_t* indices, void* out,
                                        uint64_t rows, uint64_t src_seg, uint64_t idx_seg, uint32_t* oob_flag,
                                        void* stream)
{
  if (rows == 0 || idx_seg == 0) {
    return CPN_OK;
  }
  if (src == nullptr || indices == nullptr || out == nullptr) {
    return CPN_ERR_NULL;
  }
  if (src_seg == 0) {
    return CPN_ERR_SHAPE;  // nothing to take from
  }
  const uint64_t align = static_cast<uint64_t>(elem_bytes);
  if ((reinterpret_cast<uintptr_t>(src) % align) != 0 || (reinterpret_cast<uintptr_t>(out) % align) != 0 ||
      (reinterpret_cast<uintptr_t>(indices) % 8) != 0) {
    return CPN_ERR_ALIGN;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (elem_bytes) {
    case 1: return cpn::launch_take<uint8_t>(src, indices, out, rows, src_seg, idx_seg, oob_flag, s);
    case 2: return cpn::launch_take<uint16_t>(src, indices, out, rows, src_seg, idx_seg, oob_flag, s);
    case 4: return cpn::launch_take<uint32_t>(src, indices, out, rows, src_seg, idx_seg, oob_flag, s);
    case 8: return cpn::launch_take<uint64_t>(src, indices, out, rows, src_seg, idx_seg, oob_flag, s);
    case 16: return cpn::launch_take<cpn::U128>(src, indices, out, rows, src_seg, idx_seg, oob_flag, s);
    default: return CPN_ERR_DTYPE;
  }
}
