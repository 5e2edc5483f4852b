// TEST INFRASTRUCTURE -- second CPU baseline, timed only by bench.py (never a checker for data
// with NaN, never part of the product).
//
// Restates the reference's CPU and OpenMP variants with the same library family they use:
// thrust_local_sort_inplace (src/cupynumeric/sort/sort_cpu.inl:52-85) loops over the rows and
// calls thrust::(stable_)sort / (stable_)sort_by_key on each, with the execution policy
// thrust::host (src/cupynumeric/sort/sort.cc:64) or thrust::omp::par
// (src/cupynumeric/sort/sort_omp.cc:65); SortImplBodyCpu copies the input and initialises the
// indices first (sort_cpu.inl:974-1025), which the Python wrapper does.  This build links
// ROCm's rocThrust host backends, not the CCCL the reference pins, so the timings stand for
// "thrust on the host", not for the reference binary.  On arithmetic keys thrust's host
// policy runs a radix sort that orders floats by bit pattern: with NaN or -0.0 in the data
// the output is not NumPy's order, which is why this file is a baseline only.
//
// Compiled by hipcc as a HIP source (rocThrust's headers need it); all code is host code.
#include <cstddef>
#include <cstdint>

#if !defined(__HIP_DEVICE_COMPILE__)
#include <thrust/execution_policy.h>
#include <thrust/functional.h>
#include <thrust/sort.h>
#include <thrust/system/omp/execution_policy.h>

namespace {

template <typename VAL, typename Policy>
void local_sort_inplace(VAL* inptr, int64_t* argptr, size_t volume, size_t sort_dim_size, bool stable, const Policy& exec)
{
  if (argptr == nullptr) {
    for (size_t start = 0; start < volume; start += sort_dim_size) {
      if (stable) {
        thrust::stable_sort(exec, inptr + start, inptr + start + sort_dim_size, thrust::less<VAL>());
      } else {
        thrust::sort(exec, inptr + start, inptr + start + sort_dim_size, thrust::less<VAL>());
      }
    }
  } else {
    for (size_t start = 0; start < volume; start += sort_dim_size) {
      if (stable) {
        thrust::stable_sort_by_key(exec, inptr + start, inptr + start + sort_dim_size, argptr + start,
                                   thrust::less<VAL>());
      } else {
        thrust::sort_by_key(exec, inptr + start, inptr + start + sort_dim_size, argptr + start, thrust::less<VAL>());
      }
    }
  }
}

template <typename VAL>
int run(void* values, int64_t* indices, size_t volume, size_t seg, int stable, int use_omp)
{
  if (use_omp) {
    local_sort_inplace(static_cast<VAL*>(values), indices, volume, seg, stable != 0, thrust::omp::par);
  } else {
    local_sort_inplace(static_cast<VAL*>(values), indices, volume, seg, stable != 0, thrust::host);
  }
  return 0;
}

}  // namespace
#endif

// dtype: enum cpn_dtype of include/cpn_sort.h; the integer and float types of 1 to 8 bytes
// except float16 (no host comparison operator in this toolchain).  `values` is sorted in
// place; `indices` (may be NULL) must hold the row positions on entry.
extern "C" int cpn_thrust_local_sort(int dtype, void* values, int64_t* indices, uint64_t volume, uint64_t seg,
                                     int stable, int use_omp)
{
#if !defined(__HIP_DEVICE_COMPILE__)
  if (seg == 0 || volume % seg != 0) {
    return -3;
  }
  switch (dtype) {
    case 0: return run<uint8_t>(values, indices, volume, seg, stable, use_omp);  // bool bytes
    case 1: return run<int8_t>(values, indices, volume, seg, stable, use_omp);
    case 2: return run<int16_t>(values, indices, volume, seg, stable, use_omp);
    case 3: return run<int32_t>(values, indices, volume, seg, stable, use_omp);
    case 4: return run<int64_t>(values, indices, volume, seg, stable, use_omp);
    case 5: return run<uint8_t>(values, indices, volume, seg, stable, use_omp);
    case 6: return run<uint16_t>(values, indices, volume, seg, stable, use_omp);
    case 7: return run<uint32_t>(values, indices, volume, seg, stable, use_omp);
    case 8: return run<uint64_t>(values, indices, volume, seg, stable, use_omp);
    case 10: return run<float>(values, indices, volume, seg, stable, use_omp);
    case 11: return run<double>(values, indices, volume, seg, stable, use_omp);
    default: return -1;
  }
#else
  return -8;
#endif
}
