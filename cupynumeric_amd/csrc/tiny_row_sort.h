// Very short rows (up to 32 elements): several rows share a wavefront, one element per lane,
// and every element finds its final position by comparing itself with the other elements of
// its row (rank = number of smaller keys + number of equal keys that come earlier), fetched
// from the neighbouring lanes with cross-lane shuffles.  One shot, no passes, no LDS traffic.
//
// Replaces, for such rows, the (segment id, value) tuple merge sort of
// src/cupynumeric/sort/thrust_sort.cuh:68-122.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "wave_row_sort.h"

namespace cpn {

// S = slots per row (power of two, >= row length); 64/S rows per wavefront.
template <typename KeyT, int CODEC, bool HAS_IDX, int S>
__global__ __launch_bounds__(256) void tiny_row_sort_kernel(const KeyT* keys_in,
                                                             KeyT* keys_out,
                                                             int64_t* idx_out,
                                                             uint32_t seg,
                                                             uint64_t rows,
                                                             int64_t index_offset,
                                                             uint32_t* status)
{
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    *status = 0;  // the workspace's status word: a per-row sort cannot fail on the device
  }
  using OW                = OrderedWords<CODEC, KeyT>;
  constexpr int NW        = OW::NW;
  constexpr int ROWS_WAVE = WAVE / S;
  static_assert(S >= 1 && S <= 32 && (S & (S - 1)) == 0, "slots per row: a power of two up to 32");

  const int lane      = threadIdx.x & (WAVE - 1);
  const uint64_t wave = static_cast<uint64_t>(blockIdx.x) * (256 / WAVE) + threadIdx.x / WAVE;
  const uint32_t slot = lane % S;          // position of this lane's element in its row
  const uint64_t row  = wave * ROWS_WAVE + lane / S;
  const bool valid    = (row < rows) && (slot < seg);
  const uint64_t base = row * seg;

  KeyT raw = KeyT{};
  uint32_t w[NW];
  if (valid) {
    raw = keys_in[base + slot];
    OW::encode(raw, w);
  } else {
#pragma unroll
    for (int n = 0; n < NW; ++n) {
      w[n] = 0;
    }
  }
  // rank among the valid elements of the row; all lanes take part in the shuffles
  uint32_t rank = 0;
#pragma unroll
  for (int j = 1; j < S; ++j) {
    const uint32_t pslot = (slot + j) % S;
    const int src        = (lane - static_cast<int>(slot)) + static_cast<int>(pslot);
    bool less = false, equal = true;  // partner compared with this element, most significant word first
#pragma unroll
    for (int n = NW - 1; n >= 0; --n) {
      const uint32_t pw = __shfl(w[n], src, WAVE);
      less              = less || (equal && pw < w[n]);
      equal             = equal && (pw == w[n]);
    }
    if (pslot < seg && (less || (equal && pslot < slot))) {
      ++rank;
    }
  }
  if (valid) {
    // the stores depend on the shuffles, hence on every load of the row: in place is safe
    if (keys_out != nullptr) {
      keys_out[base + rank] = raw;
    }
    if constexpr (HAS_IDX) {
      idx_out[base + rank] = static_cast<int64_t>(slot) + index_offset;
    }
  }
}

}  // namespace cpn
