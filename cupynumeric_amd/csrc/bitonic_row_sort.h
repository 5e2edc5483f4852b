// Rows of up to 64 elements, real keys of up to 8 bytes: one element per lane, 64/S rows per
// wavefront (S = slots per row, the next power of two), sorted by a bitonic network of
// compare-exchanges between lanes.  What is compared is (order-preserving image of the key,
// position in the row) as one unsigned word (an image and a position word for 8-byte keys), so
// that no two are equal: the network, which is not stable by itself, then yields exactly the
// stable order (NaNs tie with each other and +0.0 with -0.0 in the image, and the position
// decides), and slots past the end of a row, which hold the largest image, sort behind every real
// element.  The raw keys do not travel: every lane fetches the key of the position that ended up
// in its slot once, at the end.  log2(S) (log2(S) + 1) / 2 exchanges of about eight vector
// instructions (twelve for 8-byte keys), no LDS memory, no passes.
//
// Stands, for such rows, where the reference sorts (segment id, value) tuples with a merge sort
// (src/cupynumeric/sort/thrust_sort.cuh:68-122).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "key_codec.h"
#include "radix_common.h"

namespace cpn {

// The value of lane (lane ^ J) of the same wavefront.
template <int J>
__device__ __forceinline__ uint32_t lane_xor(uint32_t v)
{
  static_assert(J == 1 || J == 2 || J == 4 || J == 8 || J == 16 || J == 32, "one bit");
  if constexpr (J == 1) {
    return static_cast<uint32_t>(__builtin_amdgcn_mov_dpp(static_cast<int>(v), 0xB1, 0xF, 0xF, true));  // quad_perm [1,0,3,2]
  } else if constexpr (J == 2) {
    return static_cast<uint32_t>(__builtin_amdgcn_mov_dpp(static_cast<int>(v), 0x4E, 0xF, 0xF, true));  // quad_perm [2,3,0,1]
  } else if constexpr (J == 8) {
    return static_cast<uint32_t>(__builtin_amdgcn_mov_dpp(static_cast<int>(v), 0x128, 0xF, 0xF, true));  // row_ror:8
  } else if constexpr (J == 4 || J == 16) {
    return static_cast<uint32_t>(__builtin_amdgcn_ds_swizzle(static_cast<int>(v), (J << 10) | 0x1F));  // xor mask within 32 lanes
  } else {
    return static_cast<uint32_t>(__shfl_xor(static_cast<int>(v), 32, WAVE));
  }
}
template <int J>
__device__ __forceinline__ uint64_t lane_xor(uint64_t v)
{
  const uint32_t lo = lane_xor<J>(static_cast<uint32_t>(v));
  const uint32_t hi = lane_xor<J>(static_cast<uint32_t>(v >> 32));
  return (static_cast<uint64_t>(hi) << 32) | lo;
}

// 8-byte keys: the image and the position side by side, compared image first.
struct ImagePos {
  uint64_t image;
  uint32_t pos;
};
template <int J>
__device__ __forceinline__ ImagePos lane_xor(ImagePos v)
{
  return ImagePos{lane_xor<J>(v.image), lane_xor<J>(v.pos)};
}
__device__ __forceinline__ bool operator<(const ImagePos& a, const ImagePos& b)
{
  return a.image < b.image || (a.image == b.image && a.pos < b.pos);
}
__device__ __forceinline__ uint32_t word_pos(uint32_t w) { return w; }
__device__ __forceinline__ uint32_t word_pos(uint64_t w) { return static_cast<uint32_t>(w); }
__device__ __forceinline__ uint32_t word_pos(const ImagePos& w) { return w.pos; }

// One compare-exchange of the network: lanes l and l ^ J; the lane of the pair that is to hold
// the smaller word is the lower one where the run of K lanes it belongs to ascends.
template <int K, int J, int S, typename W>
__device__ __forceinline__ W bitonic_exchange(W w, uint32_t lane)
{
  const W other        = lane_xor<J>(w);
  const bool ascending = (K == S) || ((lane & K) == 0);  // the last merge of a row ascends in every row of the wave
  const bool lower     = (lane & J) == 0;
  const bool keep_min  = lower == ascending;
  return ((w < other) == keep_min) ? w : other;
}
template <int K, int J, int S, typename W>
__device__ __forceinline__ W bitonic_merge(W w, uint32_t lane)
{
  if constexpr (J >= 1) {
    w = bitonic_exchange<K, J, S>(w, lane);
    if constexpr (J > 1) {
      w = bitonic_merge<K, J / 2, S>(w, lane);
    }
  }
  return w;
}
template <int K, int S, typename W>
__device__ __forceinline__ W bitonic_sort(W w, uint32_t lane)
{
  if constexpr (K <= S) {
    w = bitonic_merge<K, K / 2, S>(w, lane);
    if constexpr (K < S) {
      w = bitonic_sort<2 * K, S>(w, lane);
    }
  }
  return w;
}

// S = slots per row (power of two, 2 ... 64, >= row length); 64/S rows per wavefront.
template <typename KeyT, int CODEC, bool HAS_IDX, int S>
__global__ __launch_bounds__(256) void bitonic_row_sort_kernel(const KeyT* __restrict__ keys_in,
                                                                KeyT* keys_out,
                                                                int64_t* __restrict__ idx_out,
                                                                uint32_t seg,
                                                                uint64_t rows,
                                                                int64_t index_offset,
                                                                uint32_t* status)
{
  static_assert(sizeof(KeyT) <= 8 && (CODEC == CODEC_UNSIGNED || CODEC == CODEC_SIGNED || CODEC == CODEC_FLOAT),
                "real keys of up to 8 bytes");
  static_assert(S >= 2 && S <= WAVE && (S & (S - 1)) == 0, "slots per row: a power of two up to 64");
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    *status = 0;  // the workspace's status word: a per-row sort cannot fail on the device
  }
  // 4-byte keys: image in the high word, position in the low one; shorter keys: image << 8 | position;
  // 8-byte keys: two registers for the image, one for the position
  using W = std::conditional_t<sizeof(KeyT) == 8, ImagePos, std::conditional_t<sizeof(KeyT) == 4, uint64_t, uint32_t>>;
  constexpr int ROWS_WAVE = WAVE / S;

  const uint32_t lane = threadIdx.x & (WAVE - 1);
  const uint64_t wave = static_cast<uint64_t>(blockIdx.x) * (256 / WAVE) + threadIdx.x / WAVE;
  const uint32_t slot = lane & (S - 1);  // position of this lane's element in its row
  const uint64_t row  = wave * ROWS_WAVE + lane / S;
  const bool valid    = (row < rows) && (slot < seg);
  const uint64_t base = row * seg;

  KeyT raw = KeyT{};
  if (valid) {
    raw = keys_in[base + slot];
  }
  const KeyT image = valid ? ordered_bits<CODEC, KeyT>(raw) : static_cast<KeyT>(~KeyT{0});
  W w;
  if constexpr (sizeof(KeyT) == 8) {
    w = ImagePos{image, slot};
  } else {
    w = (static_cast<W>(image) << (sizeof(KeyT) == 4 ? 32 : 8)) | slot;
  }
  w = bitonic_sort<2, S>(w, lane);

  const uint32_t from = word_pos(w) & (S - 1);  // the position whose element belongs in this slot
  const int src_lane  = static_cast<int>((lane & ~(S - 1)) | from);
  KeyT bits;
  if constexpr (sizeof(KeyT) == 8) {
    const uint32_t lo = static_cast<uint32_t>(__shfl(static_cast<int>(static_cast<uint32_t>(raw)), src_lane, WAVE));
    const uint32_t hi = static_cast<uint32_t>(__shfl(static_cast<int>(static_cast<uint32_t>(raw >> 32)), src_lane, WAVE));
    bits              = (static_cast<uint64_t>(hi) << 32) | lo;
  } else {
    bits = static_cast<KeyT>(__shfl(static_cast<int>(static_cast<uint32_t>(raw)), src_lane, WAVE));
  }
  if (valid) {  // (the first seg slots of a row hold its seg elements)
    if (keys_out != nullptr) {
      keys_out[base + slot] = bits;
    }
    if constexpr (HAS_IDX) {
      idx_out[base + slot] = static_cast<int64_t>(from) + index_offset;
    }
  }
}

}  // namespace cpn
