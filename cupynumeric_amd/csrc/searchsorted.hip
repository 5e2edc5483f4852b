// searchsorted: for every value, the leftmost ('left') or rightmost ('right') position at
// which it can be inserted into a sorted 1-D array without breaking the order.
//
// Replaces SearchSortedTask's GPU variant (src/cupynumeric/sort/searchsorted.cu:27-116: one
// thread per value, cub::LowerBound / cub::UpperBound over the sorted array, the position
// folded into the output with a MIN / MAX reduction because the sorted array may be split
// over several processors; on one GPU the bound itself is the answer).  Comparisons use the
// ordered keys of key_codec.h, i.e. the order the sort kernels produce (NaN last and equal to
// itself, -0.0 == +0.0, complex by NumPy's rule), where the reference compares with `<`.
//
// A probe of the sorted array is a dependent load, so the first eleven steps of every search
// run over a table of up to 2048 evenly spaced elements that each workgroup stages in LDS;
// the remaining steps stay inside one stride of the array.
//
// Every remaining probe of an unordered value is a sector of its own from HBM.  When the
// array is too large for the caches and there are many values, the values are therefore
// sorted first (with their positions, by the library's own sort, in the caller's workspace):
// neighbouring lanes then search for neighbouring values, their probes fall into the same
// cache lines, and the array is read about once instead of once per probe.  The answers go
// back to the positions the values came from.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "sort_driver.h"

namespace cpn {

constexpr int SEARCH_BLOCK  = 256;
constexpr int SEARCH_PIVOTS = 2048;

template <int NW>
__device__ __forceinline__ bool words_less(const uint64_t (&a)[NW], const uint64_t (&b)[NW])
{
  bool lt = false, eq = true;  // most significant word last in the array
#pragma unroll
  for (int n = NW - 1; n >= 0; --n) {
    lt = lt || (eq && a[n] < b[n]);
    eq = eq && (a[n] == b[n]);
  }
  return lt;
}

// true when the search has to continue to the right of an element with key `a`
template <bool LEFT, int NW>
__device__ __forceinline__ bool go_right(const uint64_t (&a)[NW], const uint64_t (&v)[NW])
{
  return LEFT ? words_less<NW>(a, v) : !words_less<NW>(v, a);
}

template <typename KeyT, int CODEC, bool LEFT>
__global__ __launch_bounds__(SEARCH_BLOCK) void searchsorted_kernel(const KeyT* __restrict__ sorted,
                                                                    uint64_t n,
                                                                    const KeyT* __restrict__ values,
                                                                    uint64_t num_values,
                                                                    int64_t* __restrict__ out,
                                                                    const int64_t* __restrict__ origin,
                                                                    uint64_t step,
                                                                    uint32_t num_pivots)
{
  using KT         = KeyTraits<CODEC, KeyT>;
  constexpr int NW = KT::NWORDS;
  __shared__ uint64_t s_pivot[NW][SEARCH_PIVOTS];

  // pivot j is element j*step of the sorted array (num_pivots == 0: table not used)
  for (uint32_t j = threadIdx.x; j < num_pivots; j += SEARCH_BLOCK) {
    uint64_t w[NW];
    KT::words(sorted[static_cast<uint64_t>(j) * step], w);
#pragma unroll
    for (int k = 0; k < NW; ++k) {
      s_pivot[k][j] = w[k];
    }
  }
  __syncthreads();

  const uint64_t stride = static_cast<uint64_t>(gridDim.x) * SEARCH_BLOCK;
  for (uint64_t i = static_cast<uint64_t>(blockIdx.x) * SEARCH_BLOCK + threadIdx.x; i < num_values; i += stride) {
    uint64_t v[NW];
    KT::words(values[i], v);
    uint64_t lo = 0, hi = n;
    if (num_pivots != 0) {
      // first pivot at which the search would not continue to the right
      uint32_t pl = 0, ph = num_pivots;
      while (pl < ph) {
        const uint32_t pm = (pl + ph) / 2;
        uint64_t a[NW];
#pragma unroll
        for (int k = 0; k < NW; ++k) {
          a[k] = s_pivot[k][pm];
        }
        if (go_right<LEFT, NW>(a, v)) {
          pl = pm + 1;
        } else {
          ph = pm;
        }
      }
      // elements up to pivot pl-1 are to the left of the answer, pivot pl is not
      lo = (pl == 0) ? 0 : static_cast<uint64_t>(pl - 1) * step + 1;
      hi = (pl == num_pivots) ? n : static_cast<uint64_t>(pl) * step;
    }
    while (lo < hi) {
      const uint64_t mid = lo + (hi - lo) / 2;
      uint64_t a[NW];
      KT::words(sorted[mid], a);
      if (go_right<LEFT, NW>(a, v)) {
        lo = mid + 1;
      } else {
        hi = mid;
      }
    }
    // `origin` (values sorted beforehand): the position the value had in the caller's array
    out[origin != nullptr ? static_cast<uint64_t>(origin[i]) : i] = static_cast<int64_t>(lo);
  }
}

template <typename KeyT, int CODEC>
static int launch_searchsorted(const void* sorted, uint64_t n, const void* values, uint64_t num_values, bool left,
                               int64_t* out, const int64_t* origin, hipStream_t stream)
{
  uint64_t step       = 0;
  uint32_t num_pivots = 0;
  if (n >= 8192 && num_values >= 2048) {
    step       = (n + SEARCH_PIVOTS - 1) / SEARCH_PIVOTS;
    num_pivots = static_cast<uint32_t>((n + step - 1) / step);
  }
  // with a pivot table every workgroup should serve a few thousand values
  const uint64_t per_block = (num_pivots != 0) ? 16 * SEARCH_BLOCK : SEARCH_BLOCK;
  uint64_t grid            = (num_values + per_block - 1) / per_block;
  if (grid > 16384) {
    grid = 16384;
  }
  ProfileScope prof("searchsorted", stream);
  if (left) {
    hipLaunchKernelGGL((searchsorted_kernel<KeyT, CODEC, true>), dim3(static_cast<uint32_t>(grid)), dim3(SEARCH_BLOCK),
                       0, stream, static_cast<const KeyT*>(sorted), n, static_cast<const KeyT*>(values), num_values, out,
                       origin, step, num_pivots);
  } else {
    hipLaunchKernelGGL((searchsorted_kernel<KeyT, CODEC, false>), dim3(static_cast<uint32_t>(grid)),
                       dim3(SEARCH_BLOCK), 0, stream, static_cast<const KeyT*>(sorted), n,
                       static_cast<const KeyT*>(values), num_values, out, origin, step, num_pivots);
  }
  CPN_HIP_TRY(hipGetLastError());
  return CPN_OK;
}

// Sorting the values first pays when the sorted array is far larger than the caches and the
// values are many; otherwise (and whenever the caller brings no workspace) values are searched
// in the order given.
static bool presort_pays(int key_bytes, uint64_t n, uint64_t num_values)
{
  return n * static_cast<uint64_t>(key_bytes) >= (64ull << 20) && num_values >= (1ull << 16);
}

struct SearchLayout {
  uint64_t sort_bytes, off_values, off_origin, total;
};

static SearchLayout search_layout(int dtype, int key_bytes, uint64_t num_values)
{
  SearchLayout L{};
  L.sort_bytes = cpn_local_sort_temp_bytes(dtype, num_values, num_values, 1, 1, 0);
  L.off_values = align_up(L.sort_bytes, WORKSPACE_ALIGN);
  L.off_origin = L.off_values + align_up(num_values * static_cast<uint64_t>(key_bytes), WORKSPACE_ALIGN);
  L.total      = L.off_origin + align_up(num_values * 8, WORKSPACE_ALIGN);
  return L;
}

}  // namespace cpn

extern "C" uint64_t cpn_searchsorted_temp_bytes(int dtype, uint64_t n, uint64_t num_values)
{
  const cpn::KeyKind k = cpn::key_kind(dtype);
  if (k.bytes == 0 || k.codec < 0 || !cpn::presort_pays(k.bytes, n, num_values)) {
    return 0;
  }
  const cpn::SearchLayout L = cpn::search_layout(dtype, k.bytes, num_values);
  return L.sort_bytes == 0 ? 0 : L.total;
}

extern "C" int cpn_searchsorted(int dtype, const void* sorted, uint64_t n, const void* values, uint64_t num_values,
                                int left, int64_t* positions_out, void* temp, uint64_t temp_bytes, void* stream)
{
  using namespace cpn;
  const KeyKind k = key_kind(dtype);
  if (k.bytes == 0 || k.codec < 0) {
    return CPN_ERR_DTYPE;
  }
  if (num_values == 0) {
    return CPN_OK;
  }
  if (values == nullptr || positions_out == nullptr || (n != 0 && sorted == nullptr)) {
    return CPN_ERR_NULL;
  }
  const uint64_t align = static_cast<uint64_t>(k.bytes);
  if ((reinterpret_cast<uintptr_t>(sorted) % align) != 0 || (reinterpret_cast<uintptr_t>(values) % align) != 0 ||
      (reinterpret_cast<uintptr_t>(positions_out) % 8) != 0) {
    return CPN_ERR_ALIGN;
  }
  const int64_t* origin = nullptr;
  if (temp != nullptr && presort_pays(k.bytes, n, num_values)) {
    const SearchLayout L = search_layout(dtype, k.bytes, num_values);
    if (L.sort_bytes != 0 && temp_bytes >= L.total) {
      if ((reinterpret_cast<uintptr_t>(temp) % WORKSPACE_ALIGN) != 0) {
        return CPN_ERR_TEMP;
      }
      unsigned char* ws = static_cast<unsigned char*>(temp);
      void* sorted_vals = ws + L.off_values;
      int64_t* where    = reinterpret_cast<int64_t*>(ws + L.off_origin);
      const int rc = cpn_local_sort(dtype, values, sorted_vals, where, num_values, num_values, 0, 1, ws, L.sort_bytes,
                                    stream);
      if (rc != CPN_OK) {
        return rc;
      }
      values = sorted_vals;
      origin = where;
    }
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  const bool l  = left != 0;
#define CPN_SEARCH_CASE(T, C) \
  return launch_searchsorted<T, C>(sorted, n, values, num_values, l, positions_out, origin, s)
  switch (k.codec) {
    case CODEC_UNSIGNED:
      switch (k.bytes) {
        case 1: CPN_SEARCH_CASE(uint8_t, CODEC_UNSIGNED);
        case 2: CPN_SEARCH_CASE(uint16_t, CODEC_UNSIGNED);
        case 4: CPN_SEARCH_CASE(uint32_t, CODEC_UNSIGNED);
        case 8: CPN_SEARCH_CASE(uint64_t, CODEC_UNSIGNED);
      }
      break;
    case CODEC_SIGNED:
      switch (k.bytes) {
        case 1: CPN_SEARCH_CASE(uint8_t, CODEC_SIGNED);
        case 2: CPN_SEARCH_CASE(uint16_t, CODEC_SIGNED);
        case 4: CPN_SEARCH_CASE(uint32_t, CODEC_SIGNED);
        case 8: CPN_SEARCH_CASE(uint64_t, CODEC_SIGNED);
      }
      break;
    case CODEC_FLOAT:
      switch (k.bytes) {
        case 2: CPN_SEARCH_CASE(uint16_t, CODEC_FLOAT);
        case 4: CPN_SEARCH_CASE(uint32_t, CODEC_FLOAT);
        case 8: CPN_SEARCH_CASE(uint64_t, CODEC_FLOAT);
      }
      break;
    case CODEC_COMPLEX:
      switch (k.bytes) {
        case 8: CPN_SEARCH_CASE(uint64_t, CODEC_COMPLEX);
        case 16: CPN_SEARCH_CASE(U128, CODEC_COMPLEX);
      }
      break;
  }
#undef CPN_SEARCH_CASE
  return CPN_ERR_DTYPE;
}
