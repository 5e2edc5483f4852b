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

// The same gather when the leading dimensions of `src` and `idx` broadcast against each other
// (NumPy's take_along_axis lets every dimension but the axis be 1 on either side): the row of the
// source and of the indices that belong to an output row follow from the row's coordinates and a
// stride per dimension, 0 where that side is broadcast.
constexpr int TAKE_MAX_LEAD = 7;
struct TakeLead {
  int ndim;
  uint64_t shape[TAKE_MAX_LEAD];       // leading dimensions of the output
  uint64_t src_stride[TAKE_MAX_LEAD];  // rows of src per step in that dimension (0: broadcast)
  uint64_t idx_stride[TAKE_MAX_LEAD];  // rows of idx per step
};

template <typename T>
__global__ __launch_bounds__(256) void take_last_axis_broadcast_kernel(const T* __restrict__ src,
                                                                        const int64_t* __restrict__ idx,
                                                                        T* __restrict__ out,
                                                                        uint64_t total,
                                                                        uint64_t src_seg,
                                                                        uint64_t idx_seg,
                                                                        TakeLead lead,
                                                                        uint32_t* oob_flag)
{
  const uint64_t stride = static_cast<uint64_t>(gridDim.x) * blockDim.x;
  bool bad              = false;
  for (uint64_t o = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x; o < total; o += stride) {
    uint64_t row = o / idx_seg;
    const uint64_t j = o - row * idx_seg;
    uint64_t src_row = 0, idx_row = 0;
    for (int d = lead.ndim - 1; d >= 0; --d) {
      const uint64_t c = row % lead.shape[d];
      row /= lead.shape[d];
      src_row += c * lead.src_stride[d];
      idx_row += c * lead.idx_stride[d];
    }
    int64_t k = idx[idx_row * idx_seg + j];
    if (k < 0) {
      k += static_cast<int64_t>(src_seg);
    }
    if (k < 0 || static_cast<uint64_t>(k) >= src_seg) {
      bad = true;
    } else {
      out[o] = src[src_row * src_seg + static_cast<uint64_t>(k)];
    }
  }
  if (bad && oob_flag != nullptr) {
    __hip_atomic_store(oob_flag, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}

template <typename T>
static int launch_take_broadcast(const void* src, const int64_t* idx, void* out, uint64_t rows, uint64_t src_seg,
                                 uint64_t idx_seg, const TakeLead& lead, uint32_t* oob_flag, hipStream_t stream)
{
  const uint64_t total = rows * idx_seg;
  uint64_t grid        = (total + 255) / 256;
  if (grid > (1u << 20)) {
    grid = 1u << 20;
  }
  ProfileScope prof("take_last_axis", stream);
  hipLaunchKernelGGL((take_last_axis_broadcast_kernel<T>), dim3(static_cast<uint32_t>(grid)), dim3(256), 0, stream,
                     static_cast<const T*>(src), idx, static_cast<T*>(out), total, src_seg, idx_seg, lead, oob_flag);
  CPN_HIP_TRY(hipGetLastError());
  return CPN_OK;
}

// ---- lexsort: several keys packed into one ------------------------------------------------
//
// A lexicographic order on keys (k_last, ..., k_0) is the order of the unsigned number whose
// bytes are the order-preserving images of the keys, most significant key on top.  Packing up
// to 8 bytes of real keys into one word turns the reference's chain of argsort +
// take_along_axis per key (cupynumeric/_module/ssc_sorting.py:423-444) into one argsort of
// the packed word; with `indices` the keys are read through the permutation found so far,
// which is the take_along_axis of the chain fused into the packing.
constexpr int PACK_MAX_KEYS = 8;

struct PackArgs {
  const void* key[PACK_MAX_KEYS];
  int bytes[PACK_MAX_KEYS];
  int codec[PACK_MAX_KEYS];
  int shift[PACK_MAX_KEYS];  // bit position of the key inside the packed word
  int num_keys;
};

__device__ __forceinline__ uint64_t ordered_image(const void* base, uint64_t i, int bytes, int codec)
{
  switch (bytes) {
    case 1: {
      const uint8_t raw = static_cast<const uint8_t*>(base)[i];
      return codec == CODEC_SIGNED ? ordered_bits<CODEC_SIGNED, uint8_t>(raw) : raw;
    }
    case 2: {
      const uint16_t raw = static_cast<const uint16_t*>(base)[i];
      return codec == CODEC_FLOAT ? ordered_bits<CODEC_FLOAT, uint16_t>(raw)
                                  : (codec == CODEC_SIGNED ? ordered_bits<CODEC_SIGNED, uint16_t>(raw) : raw);
    }
    case 4: {
      const uint32_t raw = static_cast<const uint32_t*>(base)[i];
      return codec == CODEC_FLOAT ? ordered_bits<CODEC_FLOAT, uint32_t>(raw)
                                  : (codec == CODEC_SIGNED ? ordered_bits<CODEC_SIGNED, uint32_t>(raw) : raw);
    }
    default: {
      const uint64_t raw = static_cast<const uint64_t*>(base)[i];
      return codec == CODEC_FLOAT ? ordered_bits<CODEC_FLOAT, uint64_t>(raw)
                                  : (codec == CODEC_SIGNED ? ordered_bits<CODEC_SIGNED, uint64_t>(raw) : raw);
    }
  }
}

template <typename OutT>
__global__ __launch_bounds__(256) void lexsort_pack_kernel(PackArgs a,
                                                            const int64_t* __restrict__ indices,
                                                            OutT* __restrict__ out,
                                                            uint64_t total,
                                                            uint64_t seg)
{
  const uint64_t stride = static_cast<uint64_t>(gridDim.x) * blockDim.x;
  for (uint64_t o = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x; o < total; o += stride) {
    uint64_t src = o;
    if (indices != nullptr) {
      src = (o / seg) * seg + static_cast<uint64_t>(indices[o]);
    }
    uint64_t packed = 0;
    for (int k = 0; k < a.num_keys; ++k) {
      packed |= ordered_image(a.key[k], src, a.bytes[k], a.codec[k]) << a.shift[k];
    }
    out[o] = static_cast<OutT>(packed);
  }
}

}  // namespace cpn

extern "C" int cpn_lexsort_pack(int num_keys, const int* dtypes, const void* const* keys, const int64_t* indices,
                                int packed_bytes, void* packed_out, uint64_t rows, uint64_t seg, void* stream)
{
  using namespace cpn;
  if (num_keys < 1 || num_keys > PACK_MAX_KEYS || (packed_bytes != 4 && packed_bytes != 8)) {
    return CPN_ERR_SHAPE;
  }
  if (dtypes == nullptr || keys == nullptr) {
    return CPN_ERR_NULL;
  }
  PackArgs a{};
  a.num_keys = num_keys;
  int bits   = 0;
  for (int k = 0; k < num_keys; ++k) {
    const KeyKind kind = key_kind(dtypes[k]);
    if (kind.bytes == 0 || kind.codec < 0 || kind.codec == CODEC_COMPLEX) {
      return CPN_ERR_DTYPE;  // complex keys do not pack: their order needs a ninth byte
    }
    if (keys[k] == nullptr && rows * seg != 0) {
      return CPN_ERR_NULL;
    }
    if ((reinterpret_cast<uintptr_t>(keys[k]) % static_cast<uint64_t>(kind.bytes)) != 0) {
      return CPN_ERR_ALIGN;
    }
    a.key[k]   = keys[k];
    a.bytes[k] = kind.bytes;
    a.codec[k] = kind.codec;
    a.shift[k] = bits;
    bits += 8 * kind.bytes;
  }
  if (bits > 8 * packed_bytes) {
    return CPN_ERR_SHAPE;
  }
  const uint64_t total = rows * seg;
  if (total == 0) {
    return CPN_OK;
  }
  if (packed_out == nullptr) {
    return CPN_ERR_NULL;
  }
  if ((reinterpret_cast<uintptr_t>(packed_out) % static_cast<uint64_t>(packed_bytes)) != 0 ||
      (reinterpret_cast<uintptr_t>(indices) % 8) != 0) {
    return CPN_ERR_ALIGN;
  }
  uint64_t grid = (total + 255) / 256;
  if (grid > (1u << 20)) {
    grid = 1u << 20;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  ProfileScope prof("lexsort_pack", s);
  if (packed_bytes == 4) {
    hipLaunchKernelGGL((lexsort_pack_kernel<uint32_t>), dim3(static_cast<uint32_t>(grid)), dim3(256), 0, s, a, indices,
                       static_cast<uint32_t*>(packed_out), total, seg);
  } else {
    hipLaunchKernelGGL((lexsort_pack_kernel<uint64_t>), dim3(static_cast<uint32_t>(grid)), dim3(256), 0, s, a, indices,
                       static_cast<uint64_t*>(packed_out), total, seg);
  }
  CPN_HIP_TRY(hipGetLastError());
  return CPN_OK;
}

extern "C" int cpn_take_along_last_axis(int elem_bytes, const void* src, const int64_t* indices, void* out,
                                        uint64_t rows, uint64_t src_seg, uint64_t idx_seg, uint32_t* oob_flag,
                                        void* stream)
{
  if (elem_bytes != 1 && elem_bytes != 2 && elem_bytes != 4 && elem_bytes != 8 && elem_bytes != 16) {
    return CPN_ERR_DTYPE;  // (before anything divides by it)
  }
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

extern "C" int cpn_take_along_last_axis_broadcast(int elem_bytes, const void* src, const int64_t* indices, void* out,
                                                  int lead_ndim, const uint64_t* out_lead_shape,
                                                  const uint64_t* src_lead_strides, const uint64_t* idx_lead_strides,
                                                  uint64_t src_seg, uint64_t idx_seg, uint32_t* oob_flag, void* stream)
{
  if (elem_bytes != 1 && elem_bytes != 2 && elem_bytes != 4 && elem_bytes != 8 && elem_bytes != 16) {
    return CPN_ERR_DTYPE;
  }
  if (lead_ndim < 0 || lead_ndim > cpn::TAKE_MAX_LEAD) {
    return CPN_ERR_SHAPE;
  }
  if (lead_ndim > 0 && (out_lead_shape == nullptr || src_lead_strides == nullptr || idx_lead_strides == nullptr)) {
    return CPN_ERR_NULL;
  }
  cpn::TakeLead lead{};
  lead.ndim     = lead_ndim;
  uint64_t rows = 1;
  for (int d = 0; d < lead_ndim; ++d) {
    lead.shape[d]      = out_lead_shape[d];
    lead.src_stride[d] = src_lead_strides[d];
    lead.idx_stride[d] = idx_lead_strides[d];
    rows *= out_lead_shape[d];
  }
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
    case 1: return cpn::launch_take_broadcast<uint8_t>(src, indices, out, rows, src_seg, idx_seg, lead, oob_flag, s);
    case 2: return cpn::launch_take_broadcast<uint16_t>(src, indices, out, rows, src_seg, idx_seg, lead, oob_flag, s);
    case 4: return cpn::launch_take_broadcast<uint32_t>(src, indices, out, rows, src_seg, idx_seg, lead, oob_flag, s);
    case 8: return cpn::launch_take_broadcast<uint64_t>(src, indices, out, rows, src_seg, idx_seg, lead, oob_flag, s);
    case 16: return cpn::launch_take_broadcast<cpn::U128>(src, indices, out, rows, src_seg, idx_seg, lead, oob_flag, s);
    default: return CPN_ERR_DTYPE;
  }
}
