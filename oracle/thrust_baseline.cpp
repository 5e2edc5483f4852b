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
// "thrust on the host", not for the reference binary.
//
// The comparator decides which host algorithm thrust runs.  The reference passes the transparent
// `::cuda::std::less{}` (sort_cpu.inl:62-83).  In rocThrust a sort of arithmetic keys becomes a
// radix sort only when the comparator is exactly thrust::less<KeyType> or thrust::greater<KeyType>
// (thrust/system/detail/sequential/sort.inl, use_primitive_sort); every other comparator, the
// transparent less<> included, takes the merge sort.  Whether the CCCL version the reference pins
// treats its transparent comparator like the typed one cannot be checked here (CCCL is not in this
// image), so both are built and timed, and named for what they ran:
//   transparent == 0   thrust::less<VAL>   radix sort (bit-pattern order: NaN and -0.0 do not land
//                                          where NumPy puts them)
//   transparent != 0   thrust::less<>      merge sort (on data with NaN the comparison is not a
//                                          strict weak order and the output is not sorted)
// which is why this file is a baseline only.
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

template <typename VAL, typename Policy, typename Compare>
void local_sort_inplace(VAL* inptr, int64_t* argptr, size_t volume, size_t sort_dim_size, bool stable, const Policy& exec,
                        Compare comp)
{
  if (argptr == nullptr) {
    for (size_t start = 0; start < volume; start += sort_dim_size) {
      if (stable) {
        thrust::stable_sort(exec, inptr + start, inptr + start + sort_dim_size, comp);
      } else {
        thrust::sort(exec, inptr + start, inptr + start + sort_dim_size, comp);
      }
    }
  } else {
    for (size_t start = 0; start < volume; start += sort_dim_size) {
      if (stable) {
        thrust::stable_sort_by_key(exec, inptr + start, inptr + start + sort_dim_size, argptr + start, comp);
      } else {
        thrust::sort_by_key(exec, inptr + start, inptr + start + sort_dim_size, argptr + start, comp);
      }
    }
  }
}

template <typename VAL, typename Compare>
void run_with(void* values, int64_t* indices, size_t volume, size_t seg, int stable, int use_omp, Compare comp)
{
  if (use_omp) {
    local_sort_inplace(static_cast<VAL*>(values), indices, volume, seg, stable != 0, thrust::omp::par, comp);
  } else {
    local_sort_inplace(static_cast<VAL*>(values), indices, volume, seg, stable != 0, thrust::host, comp);
  }
}

template <typename VAL>
int run(void* values, int64_t* indices, size_t volume, size_t seg, int stable, int use_omp, int transparent)
{
  if (transparent) {
    run_with<VAL>(values, indices, volume, seg, stable, use_omp, thrust::less<>());
  } else {
    run_with<VAL>(values, indices, volume, seg, stable, use_omp, thrust::less<VAL>());
  }
  return 0;
}

}  // namespace
#endif

// dtype: enum cpn_dtype of include/cpn_sort.h; the integer and float types of 1 to 8 bytes
// except float16 (no host comparison operator in this toolchain).  `values` is sorted in
// place; `indices` (may be NULL) must hold the row positions on entry.  `transparent`: which
// comparator, see the head of this file.
extern "C" int cpn_thrust_local_sort(int dtype, void* values, int64_t* indices, uint64_t volume, uint64_t seg,
                                     int stable, int use_omp, int transparent)
{
#if !defined(__HIP_DEVICE_COMPILE__)
  if (seg == 0 || volume % seg != 0) {
    return -3;
  }
  switch (dtype) {
    case 0: return run<uint8_t>(values, indices, volume, seg, stable, use_omp, transparent);  // bool bytes
    case 1: return run<int8_t>(values, indices, volume, seg, stable, use_omp, transparent);
    case 2: return run<int16_t>(values, indices, volume, seg, stable, use_omp, transparent);
    case 3: return run<int32_t>(values, indices, volume, seg, stable, use_omp, transparent);
    case 4: return run<int64_t>(values, indices, volume, seg, stable, use_omp, transparent);
    case 5: return run<uint8_t>(values, indices, volume, seg, stable, use_omp, transparent);
    case 6: return run<uint16_t>(values, indices, volume, seg, stable, use_omp, transparent);
    case 7: return run<uint32_t>(values, indices, volume, seg, stable, use_omp, transparent);
    case 8: return run<uint64_t>(values, indices, volume, seg, stable, use_omp, transparent);
    case 10: return run<float>(values, indices, volume, seg, stable, use_omp, transparent);
    case 11: return run<double>(values, indices, volume, seg, stable, use_omp, transparent);
    default: return -1;
  }
#else
  return -8;
#endif
}
