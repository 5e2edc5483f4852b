// unique: the sorted distinct values of an array.
//
// Replaces UniqueTask's GPU variant on one processor (src/cupynumeric/set/unique.cu:137-204:
// copy into a buffer, thrust::sort, thrust::unique, result handed back as an unbound store of
// the distinct count; the tree reduction over ranks :49-135 belongs to the multi-GPU case).
// Here: the library's own stable sort into the workspace, then a compaction that keeps the
// first element of every run of equal keys.  Equality is equality of the ordered keys of
// key_codec.h: all NaNs are one value, -0.0 and +0.0 are one value, and every complex number
// with a NaN part is one value, as for numpy.unique (equal_nan=True), whereas thrust::unique
// compares with == and keeps every NaN.
//
// Compaction in three launches: heads per 4096-element tile, exclusive scan of the tile
// counts by one workgroup, scatter.  The sorted buffer is read twice and the output written
// once; the number of distinct values ends up in device memory and the caller reads it.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "sort_driver.h"

namespace cpn {

constexpr int UNIQUE_BLOCK = 256;
constexpr int UNIQUE_ITEMS = 16;
constexpr int UNIQUE_TILE  = UNIQUE_BLOCK * UNIQUE_ITEMS;
constexpr int UNIQUE_WAVES = UNIQUE_BLOCK / WAVE;

template <typename KeyT, int CODEC>
__device__ __forceinline__ bool starts_run(const KeyT* __restrict__ sorted, uint64_t i)
{
  using KT = KeyTraits<CODEC, KeyT>;
  if (i == 0) {
    return true;
  }
  uint64_t a[KT::NWORDS], b[KT::NWORDS];
  KT::words(sorted[i], a);
  KT::words(sorted[i - 1], b);
  bool differ = false;
#pragma unroll
  for (int k = 0; k < KT::NWORDS; ++k) {
    differ = differ || (a[k] != b[k]);
  }
  if constexpr (CODEC == CODEC_COMPLEX) {
    // the most significant word is the NaN class (0 = no NaN part): the NaN classes sort last
    // and form one value
    if (a[KT::NWORDS - 1] != 0 && b[KT::NWORDS - 1] != 0) {
      differ = false;
    }
  }
  return differ;
}

// counts[b] = number of run heads in tile b
template <typename KeyT, int CODEC>
__global__ __launch_bounds__(UNIQUE_BLOCK) void unique_count_kernel(const KeyT* __restrict__ sorted,
                                                                    uint64_t n,
                                                                    uint64_t* __restrict__ counts)
{
  __shared__ uint32_t s_wave[UNIQUE_WAVES];
  const uint64_t base = static_cast<uint64_t>(blockIdx.x) * UNIQUE_TILE;
  uint32_t cnt        = 0;
#pragma unroll 4
  for (int it = 0; it < UNIQUE_ITEMS; ++it) {
    const uint64_t i = base + static_cast<uint64_t>(it) * UNIQUE_BLOCK + threadIdx.x;
    if (i < n && starts_run<KeyT, CODEC>(sorted, i)) {
      ++cnt;
    }
  }
#pragma unroll
  for (int delta = WAVE / 2; delta > 0; delta >>= 1) {
    cnt += __shfl_xor(cnt, delta, WAVE);
  }
  if ((threadIdx.x & (WAVE - 1)) == 0) {
    s_wave[threadIdx.x / WAVE] = cnt;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    uint32_t total = 0;
#pragma unroll
    for (int w = 0; w < UNIQUE_WAVES; ++w) {
      total += s_wave[w];
    }
    counts[blockIdx.x] = total;
  }
}

// counts[0..tiles) -> exclusive prefix sums in place; the grand total goes to counts[tiles]
// and to *total_out.  One workgroup.
__global__ __launch_bounds__(1024) void unique_scan_kernel(uint64_t* counts, uint64_t tiles, uint64_t* total_out)
{
  __shared__ uint64_t s_wave[1024 / WAVE];
  __shared__ uint64_t s_carry;
  const int lane = threadIdx.x & (WAVE - 1);
  const int wave = threadIdx.x / WAVE;
  if (threadIdx.x == 0) {
    s_carry = 0;
  }
  __syncthreads();
  for (uint64_t start = 0; start < tiles; start += 1024) {
    const uint64_t i = start + threadIdx.x;
    const uint64_t c = (i < tiles) ? counts[i] : 0;
    uint64_t incl    = c;
#pragma unroll
    for (int delta = 1; delta < WAVE; delta <<= 1) {
      const uint64_t t = __shfl_up(incl, delta, WAVE);
      if (lane >= delta) {
        incl += t;
      }
    }
    if (lane == WAVE - 1) {
      s_wave[wave] = incl;
    }
    __syncthreads();
    uint64_t before = s_carry;
    for (int w = 0; w < wave; ++w) {
      before += s_wave[w];
    }
    if (i < tiles) {
      counts[i] = before + incl - c;
    }
    __syncthreads();
    if (threadIdx.x == 1023) {
      s_carry = before + incl;
    }
    __syncthreads();
  }
  if (threadIdx.x == 0) {
    counts[tiles] = s_carry;
    *total_out    = s_carry;
  }
}

template <typename KeyT, int CODEC>
__global__ __launch_bounds__(UNIQUE_BLOCK) void unique_scatter_kernel(const KeyT* __restrict__ sorted,
                                                                      uint64_t n,
                                                                      const uint64_t* __restrict__ offsets,
                                                                      KeyT* __restrict__ out)
{
  __shared__ uint32_t s_cnt[UNIQUE_ITEMS * UNIQUE_WAVES];
  const int lane      = threadIdx.x & (WAVE - 1);
  const int wave      = threadIdx.x / WAVE;
  const uint64_t base = static_cast<uint64_t>(blockIdx.x) * UNIQUE_TILE;
  uint32_t heads      = 0;  // bit it: this thread's element of round it starts a run
  uint32_t below[UNIQUE_ITEMS];
#pragma unroll
  for (int it = 0; it < UNIQUE_ITEMS; ++it) {
    const uint64_t i   = base + static_cast<uint64_t>(it) * UNIQUE_BLOCK + threadIdx.x;
    const bool head    = (i < n) && starts_run<KeyT, CODEC>(sorted, i);
    const uint64_t bal = __builtin_amdgcn_ballot_w64(head);
    below[it]          = lanes_below(bal);
    heads |= head ? (1u << it) : 0u;
    if (lane == 0) {
      s_cnt[it * UNIQUE_WAVES + wave] = static_cast<uint32_t>(__builtin_popcountll(bal));
    }
  }
  __syncthreads();
  // element order inside the tile is (round, wave, lane): scan the 64 counts in that order
  if (wave == 0) {
    const uint32_t c    = s_cnt[lane];
    const uint32_t incl = wave_inclusive_scan(c, lane);
    s_cnt[lane]         = incl - c;
  }
  __syncthreads();
  const uint64_t tile_off = offsets[blockIdx.x];
#pragma unroll
  for (int it = 0; it < UNIQUE_ITEMS; ++it) {
    if ((heads >> it) & 1u) {
      const uint64_t i = base + static_cast<uint64_t>(it) * UNIQUE_BLOCK + threadIdx.x;
      out[tile_off + s_cnt[it * UNIQUE_WAVES + wave] + below[it]] = sorted[i];
    }
  }
}
static_assert(UNIQUE_ITEMS * UNIQUE_WAVES == WAVE, "one wave scans the per-round counts");

struct UniqueLayout {
  uint64_t sort_bytes;
  uint64_t off_sorted;
  uint64_t off_counts;
  uint64_t total;
  uint64_t tiles;
};

static UniqueLayout unique_layout(int dtype, uint64_t volume)
{
  UniqueLayout L{};
  const KeyKind k = key_kind(dtype);
  L.sort_bytes    = cpn_local_sort_temp_bytes(dtype, volume, volume, 1, 0, 0);
  L.tiles         = (volume + UNIQUE_TILE - 1) / UNIQUE_TILE;
  L.off_sorted    = align_up(L.sort_bytes, WORKSPACE_ALIGN);
  L.off_counts    = L.off_sorted + align_up(volume * static_cast<uint64_t>(k.bytes), WORKSPACE_ALIGN);
  L.total         = L.off_counts + align_up((L.tiles + 1) * 8, WORKSPACE_ALIGN);
  return L;
}

template <typename KeyT, int CODEC>
static int compact(const void* sorted, uint64_t n, uint64_t* counts, uint64_t tiles, void* out, uint64_t* count_out,
                   hipStream_t stream)
{
  if (tiles >= (1ull << 31)) {
    return CPN_ERR_UNSUPPORTED;
  }
  {
    ProfileScope prof("unique_count", stream);
    hipLaunchKernelGGL((unique_count_kernel<KeyT, CODEC>), dim3(static_cast<uint32_t>(tiles)), dim3(UNIQUE_BLOCK), 0,
                       stream, static_cast<const KeyT*>(sorted), n, counts);
  }
  CPN_HIP_TRY(hipGetLastError());
  {
    ProfileScope prof("unique_scan", stream);
    hipLaunchKernelGGL(unique_scan_kernel, dim3(1), dim3(1024), 0, stream, counts, tiles, count_out);
  }
  CPN_HIP_TRY(hipGetLastError());
  {
    ProfileScope prof("unique_scatter", stream);
    hipLaunchKernelGGL((unique_scatter_kernel<KeyT, CODEC>), dim3(static_cast<uint32_t>(tiles)), dim3(UNIQUE_BLOCK), 0,
                       stream, static_cast<const KeyT*>(sorted), n, counts, static_cast<KeyT*>(out));
  }
  CPN_HIP_TRY(hipGetLastError());
  return CPN_OK;
}

}  // namespace cpn

extern "C" uint64_t cpn_unique_temp_bytes(int dtype, uint64_t volume)
{
  const cpn::KeyKind k = cpn::key_kind(dtype);
  if (k.bytes == 0 || k.codec < 0) {
    return 0;
  }
  if (volume == 0) {
    return cpn::HEADER_BYTES;
  }
  const cpn::UniqueLayout L = cpn::unique_layout(dtype, volume);
  return L.sort_bytes == 0 ? 0 : L.total;
}

extern "C" int cpn_unique(int dtype, const void* values_in, void* values_out, uint64_t volume, uint64_t* count_out,
                          void* temp, uint64_t temp_bytes, void* stream)
{
  using namespace cpn;
  const KeyKind k = key_kind(dtype);
  if (k.bytes == 0 || k.codec < 0) {
    return CPN_ERR_DTYPE;
  }
  if (count_out == nullptr) {
    return CPN_ERR_NULL;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (volume == 0) {
    // *count_out = 0 through the fill kernel (the word may be captured into a graph)
    if ((reinterpret_cast<uintptr_t>(count_out) % 8) != 0) {
      return CPN_ERR_ALIGN;
    }
    hipLaunchKernelGGL(unique_scan_kernel, dim3(1), dim3(1024), 0, s, count_out, uint64_t{0}, count_out);
    CPN_HIP_TRY(hipGetLastError());
    return CPN_OK;
  }
  if (values_in == nullptr || values_out == nullptr) {
    return CPN_ERR_NULL;
  }
  const UniqueLayout L = unique_layout(dtype, volume);
  if (L.sort_bytes == 0) {
    return CPN_ERR_UNSUPPORTED;
  }
  if (temp == nullptr || temp_bytes < L.total || (reinterpret_cast<uintptr_t>(temp) % WORKSPACE_ALIGN) != 0) {
    return CPN_ERR_TEMP;
  }
  if ((reinterpret_cast<uintptr_t>(count_out) % 8) != 0) {
    return CPN_ERR_ALIGN;
  }
  unsigned char* ws = static_cast<unsigned char*>(temp);
  void* sorted      = ws + L.off_sorted;
  uint64_t* counts  = reinterpret_cast<uint64_t*>(ws + L.off_counts);
  int rc = cpn_local_sort(dtype, values_in, sorted, nullptr, volume, volume, 0, 1, ws, L.sort_bytes, stream);
  if (rc != CPN_OK) {
    return rc;
  }
#define CPN_UNIQUE_CASE(T, C) return compact<T, C>(sorted, volume, counts, L.tiles, values_out, count_out, s)
  switch (k.codec) {
    case CODEC_UNSIGNED:
      switch (k.bytes) {
        case 1: CPN_UNIQUE_CASE(uint8_t, CODEC_UNSIGNED);
        case 2: CPN_UNIQUE_CASE(uint16_t, CODEC_UNSIGNED);
        case 4: CPN_UNIQUE_CASE(uint32_t, CODEC_UNSIGNED);
        case 8: CPN_UNIQUE_CASE(uint64_t, CODEC_UNSIGNED);
      }
      break;
    case CODEC_SIGNED:
      // equality of signed keys is equality of their bits
      switch (k.bytes) {
        case 1: CPN_UNIQUE_CASE(uint8_t, CODEC_UNSIGNED);
        case 2: CPN_UNIQUE_CASE(uint16_t, CODEC_UNSIGNED);
        case 4: CPN_UNIQUE_CASE(uint32_t, CODEC_UNSIGNED);
        case 8: CPN_UNIQUE_CASE(uint64_t, CODEC_UNSIGNED);
      }
      break;
    case CODEC_FLOAT:
      switch (k.bytes) {
        case 2: CPN_UNIQUE_CASE(uint16_t, CODEC_FLOAT);
        case 4: CPN_UNIQUE_CASE(uint32_t, CODEC_FLOAT);
        case 8: CPN_UNIQUE_CASE(uint64_t, CODEC_FLOAT);
      }
      break;
    case CODEC_COMPLEX:
      switch (k.bytes) {
        case 8: CPN_UNIQUE_CASE(uint64_t, CODEC_COMPLEX);
        case 16: CPN_UNIQUE_CASE(U128, CODEC_COMPLEX);
      }
      break;
  }
#undef CPN_UNIQUE_CASE
  return CPN_ERR_DTYPE;
}
