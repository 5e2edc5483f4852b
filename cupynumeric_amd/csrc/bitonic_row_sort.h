// Rows of up to 64 elements of real keys of up to 8 bytes, one element per lane and 64/S rows per
// wavefront (S = slots per row, the next power of two), and rows of 65 ... 128 such keys, two
// elements per lane and one row per wavefront, sorted by a bitonic network of
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

// 8-byte keys: the image and the position side by side, compared image first.  Two elements per
// lane (rows of 65 ... 128) pay off for them as well once the select between two words is written
// member by member (below): 2^26 float64 keys in rows of 128 0.49 ms through the ranking kernel,
// 0.42 ms here (0.62 ms while the select went through memory).
struct ImagePos {
  uint64_t image;
  uint64_t pos;  // (64 bits so that the struct has no padding; 32 of them travel)
};
template <int J>
__device__ __forceinline__ ImagePos lane_xor(ImagePos v)
{
  return ImagePos{lane_xor<J>(v.image), lane_xor<J>(static_cast<uint32_t>(v.pos))};
}
__device__ __forceinline__ bool operator<(const ImagePos& a, const ImagePos& b)
{
  return a.image < b.image || (a.image == b.image && static_cast<uint32_t>(a.pos) < static_cast<uint32_t>(b.pos));
}
// (member by member: a select between two structs goes through their addresses, i.e. through memory)
__device__ __forceinline__ ImagePos word_select(bool first, const ImagePos& a, const ImagePos& b)
{
  return ImagePos{first ? a.image : b.image, first ? a.pos : b.pos};
}
__device__ __forceinline__ uint32_t word_select(bool first, uint32_t a, uint32_t b) { return first ? a : b; }
__device__ __forceinline__ uint64_t word_select(bool first, uint64_t a, uint64_t b) { return first ? a : b; }
__device__ __forceinline__ uint32_t word_pos(uint32_t w) { return w; }
__device__ __forceinline__ uint32_t word_pos(uint64_t w) { return static_cast<uint32_t>(w); }
__device__ __forceinline__ uint32_t word_pos(const ImagePos& w) { return static_cast<uint32_t>(w.pos); }

// One step of the network on rows of N = 64 E elements, element i of a row in register i / 64 of
// lane i % 64 (E == 1: S <= 64 slots per row and 64 / S rows per wavefront): element i meets
// element i ^ J, and the one of the two that is to hold the smaller word is the lower one where
// the run of K elements it belongs to ascends.  J < 64 exchanges between lanes, J >= 64 between
// the registers of a lane.
template <int K, int J, int N, int E, typename W>
__device__ __forceinline__ void bitonic_exchange(W (&w)[E], uint32_t lane)
{
  if constexpr (J < WAVE) {
    const bool lower = (lane & J) == 0;
#pragma unroll
    for (int e = 0; e < E; ++e) {
      const W other = lane_xor<J>(w[e]);
      // (the last merge of a row ascends in every row of the wave)
      const bool ascending = (K == N) || (K < WAVE ? (lane & K) == 0 : ((e * WAVE) & K) == 0);
      const bool keep_min  = lower == ascending;
      w[e]                 = word_select((w[e] < other) == keep_min, w[e], other);
    }
  } else {
    constexpr int D = J / WAVE;
#pragma unroll
    for (int e = 0; e < E; ++e) {
      if ((e & D) == 0) {
        const bool ascending = (K == N) || (((e * WAVE) & K) == 0);
        const W a = w[e], b = w[e + D];
        const bool swap = (b < a) == ascending;
        w[e]            = word_select(swap, b, a);
        w[e + D]        = word_select(swap, a, b);
      }
    }
  }
}
template <int K, int J, int N, int E, typename W>
__device__ __forceinline__ void bitonic_merge(W (&w)[E], uint32_t lane)
{
  if constexpr (J >= 1) {
    bitonic_exchange<K, J, N>(w, lane);
    if constexpr (J > 1) {
      bitonic_merge<K, J / 2, N>(w, lane);
    }
  }
}
template <int K, int N, int E, typename W>
__device__ __forceinline__ void bitonic_sort(W (&w)[E], uint32_t lane)
{
  if constexpr (K <= N) {
    bitonic_merge<K, K / 2, N>(w, lane);
    if constexpr (K < N) {
      bitonic_sort<2 * K, N>(w, lane);
    }
  }
}

// S = slots per row (power of two, 2 ... 128, >= row length); 64/S rows per wavefront up to 64
// slots, one row per wavefront and two elements per lane for 128.
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
  static_assert(S >= 2 && S <= 2 * WAVE && (S & (S - 1)) == 0, "slots per row: a power of two up to 128");

  if (blockIdx.x == 0 && threadIdx.x == 0) {
    *status = 0;  // the workspace's status word: a per-row sort cannot fail on the device
  }
  // 4-byte keys: image in the high word, position in the low one; shorter keys: image << 8 | position;
  // 8-byte keys: two registers for the image, one for the position
  using W = std::conditional_t<sizeof(KeyT) == 8, ImagePos, std::conditional_t<sizeof(KeyT) == 4, uint64_t, uint32_t>>;
  constexpr int E         = S > WAVE ? S / WAVE : 1;  // elements per lane
  constexpr int LANES     = S > WAVE ? WAVE : S;      // lanes per row
  constexpr int ROWS_WAVE = WAVE / LANES;

  const uint32_t lane = threadIdx.x & (WAVE - 1);
  const uint64_t wave = static_cast<uint64_t>(blockIdx.x) * (256 / WAVE) + threadIdx.x / WAVE;
  const uint32_t slot = lane & (LANES - 1);  // position of this lane's first element in its row
  const uint64_t row  = wave * ROWS_WAVE + lane / LANES;
  const uint64_t base = row * seg;

  KeyT raw[E];
  W w[E];
#pragma unroll
  for (int e = 0; e < E; ++e) {  // (all loads first)
    const uint32_t pos = slot + e * WAVE;
    const bool valid   = (row < rows) && (pos < seg);
    raw[e]             = KeyT{};
    if (valid) {
      raw[e] = keys_in[base + pos];
    }
  }
#pragma unroll
  for (int e = 0; e < E; ++e) {
    const uint32_t pos = slot + e * WAVE;
    const bool valid   = (row < rows) && (pos < seg);
    const KeyT image   = valid ? ordered_bits<CODEC, KeyT>(raw[e]) : static_cast<KeyT>(~KeyT{0});
    if constexpr (sizeof(KeyT) == 8) {
      w[e] = ImagePos{image, pos};
    } else {
      w[e] = (static_cast<W>(image) << (sizeof(KeyT) == 4 ? 32 : 8)) | pos;
    }
  }
  bitonic_sort<2, S>(w, lane);

#pragma unroll
  for (int e = 0; e < E; ++e) {
    const uint32_t pos  = slot + e * WAVE;
    const uint32_t from = word_pos(w[e]) & (S - 1);  // the position whose element belongs here
    const int src_lane  = static_cast<int>((lane & ~(LANES - 1)) | (from & (LANES - 1)));
    KeyT bits           = KeyT{};
#pragma unroll
    for (int f = 0; f < E; ++f) {  // the register of that lane that holds it
      KeyT got;
      if constexpr (sizeof(KeyT) == 8) {
        const uint32_t lo = static_cast<uint32_t>(__shfl(static_cast<int>(static_cast<uint32_t>(raw[f])), src_lane, WAVE));
        const uint32_t hi = static_cast<uint32_t>(__shfl(static_cast<int>(static_cast<uint32_t>(raw[f] >> 32)), src_lane, WAVE));
        got               = (static_cast<uint64_t>(hi) << 32) | lo;
      } else {
        got = static_cast<KeyT>(__shfl(static_cast<int>(static_cast<uint32_t>(raw[f])), src_lane, WAVE));
      }
      bits = (E == 1 || from / WAVE == static_cast<uint32_t>(f)) ? got : bits;
    }
    if ((row < rows) && (pos < seg)) {  // (the first seg positions of a row hold its seg elements)
      if (keys_out != nullptr) {
        keys_out[base + pos] = bits;
      }
      if constexpr (HAS_IDX) {
        idx_out[base + pos] = static_cast<int64_t>(from) + index_offset;
      }
    }
  }
}

}  // namespace cpn
