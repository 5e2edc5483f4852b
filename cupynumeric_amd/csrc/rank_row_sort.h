// Rows of a few dozen real keys whose length is not a power of two: every element finds its final
// position by counting the elements of its row that come before it (smaller keys, and equal keys of
// lower position, which is the stable order).  The rows of a workgroup lie back to back in LDS as
// order-preserving images, two elements per thread whatever the row length, so no lane idles as it
// does in a network of the next power of two of slots (bitonic_row_sort.h: a row of 33 keys costs
// what a row of 64 does there).  A step of the count is one LDS read that the lanes of a row share,
// one or two compares and an add; n steps per key, so this pays for short rows only.
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

constexpr int RANK_ROW_BLOCK = 256;

// Threads that share a row: every thread holds two of its elements, h and h + ceil(seg / 2), so that one
// LDS read of a step serves two counts.
__host__ __device__ constexpr uint32_t rank_row_threads(uint32_t seg) { return (seg + 1) / 2; }

// grid = ceil(rows / rows_per_block), rows_per_block = RANK_ROW_BLOCK / rank_row_threads(seg) (seg <= 512).
template <typename KeyT, int CODEC, bool HAS_IDX>
__global__ __launch_bounds__(RANK_ROW_BLOCK) void rank_row_sort_kernel(const KeyT* keys_in,
                                                                        KeyT* keys_out,
                                                                        int64_t* idx_out,
                                                                        uint32_t seg,
                                                                        uint64_t rows,
                                                                        uint32_t rows_per_block,
                                                                        int64_t index_offset,
                                                                        uint32_t* status)
{
  static_assert(sizeof(KeyT) <= 8 && (CODEC == CODEC_UNSIGNED || CODEC == CODEC_SIGNED || CODEC == CODEC_FLOAT),
                "real keys of up to 8 bytes");
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    *status = 0;  // the workspace's status word: a per-row sort cannot fail on the device
  }
  // What is compared, as one unsigned word in which no two elements of a row are equal: keys of up to
  // 2 bytes as image << 16 | position in 32 bits (held that way in LDS); 4-byte keys as
  // image << 32 | position in 64 bits (LDS holds the image, the position is the step's number);
  // 8-byte keys as the image, with the position deciding ties.
  using ImgT = typename std::conditional<sizeof(KeyT) == 8, uint64_t, uint32_t>::type;
  constexpr bool PACKED = sizeof(KeyT) <= 2;
  constexpr int MAX_ELEMS = 2 * RANK_ROW_BLOCK;
  __shared__ ImgT s_img[MAX_ELEMS];

  const uint32_t tid    = threadIdx.x;
  const uint32_t half   = rank_row_threads(seg);
  const uint32_t local  = tid / half;  // row of this thread inside the workgroup
  const uint32_t h      = tid - local * half;
  const uint64_t row    = static_cast<uint64_t>(blockIdx.x) * rows_per_block + local;
  const bool in_row     = (local < rows_per_block) && (row < rows);
  const uint64_t base   = row * seg;
  const uint32_t pos[2] = {h, h + half};
  const bool valid[2]   = {in_row, in_row && (h + half < seg)};

  KeyT raw[2];
  ImgT image[2];
#pragma unroll
  for (int e = 0; e < 2; ++e) {
    raw[e] = KeyT{};
    if (valid[e]) {
      raw[e] = keys_in[base + pos[e]];
    }
  }
#pragma unroll
  for (int e = 0; e < 2; ++e) {
    image[e] = PACKED ? ((static_cast<ImgT>(ordered_bits<CODEC, KeyT>(raw[e])) << 16) | pos[e])
                      : static_cast<ImgT>(ordered_bits<CODEC, KeyT>(raw[e]));
    if (valid[e]) {
      s_img[local * seg + pos[e]] = image[e];
    }
  }
  __syncthreads();  // (also: every element of the workgroup's rows has been read, so sorting in place is safe)

  const ImgT* mine = s_img + (in_row ? local * seg : 0u);
  uint32_t rank[2] = {0u, 0u};
  if constexpr (sizeof(KeyT) == 4) {
    const uint64_t w0 = (static_cast<uint64_t>(image[0]) << 32) | pos[0];
    const uint64_t w1 = (static_cast<uint64_t>(image[1]) << 32) | pos[1];
#pragma unroll 8
    for (uint32_t j = 0; j < seg; ++j) {
      const uint64_t other = (static_cast<uint64_t>(mine[j]) << 32) | j;
      rank[0] += (other < w0) ? 1u : 0u;
      rank[1] += (other < w1) ? 1u : 0u;
    }
  } else {
#pragma unroll 8
    for (uint32_t j = 0; j < seg; ++j) {
      const ImgT other = mine[j];
#pragma unroll
      for (int e = 0; e < 2; ++e) {
        if constexpr (PACKED) {
          rank[e] += (other < image[e]) ? 1u : 0u;
        } else {
          rank[e] += ((other < image[e]) | ((other == image[e]) & (j < pos[e]))) ? 1u : 0u;
        }
      }
    }
  }
#pragma unroll
  for (int e = 0; e < 2; ++e) {
    if (valid[e]) {
      if (keys_out != nullptr) {
        keys_out[base + rank[e]] = raw[e];
      }
      if constexpr (HAS_IDX) {
        idx_out[base + rank[e]] = static_cast<int64_t>(pos[e]) + index_offset;
      }
    }
  }
}

}  // namespace cpn
