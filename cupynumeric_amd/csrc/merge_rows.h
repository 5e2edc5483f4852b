// Rows a little too long for the per-row kernels: every row is sorted as two halves by the
// one-workgroup-per-row kernel (each half fits the LDS of a CU) and the halves are merged here.
// One read and one write of HBM per element and step, against one pass per key byte, per-row
// histograms and tiles that end at every row on the global path.
//
// Stands, for rows of up to twice the LDS capacity, where the reference runs
// cub::DeviceSegmentedRadixSort (src/cupynumeric/sort/cub_sort.cuh:81-105,153-182).
//
// The merge is stable: of two keys that tie, the one from the first half (the lower positions of
// the row) comes first, and inside a half the stable row sort has kept input order.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "key_codec.h"
#include "radix_common.h"

namespace cpn {

constexpr int MERGE_ITEMS = 8;
// Threads of a workgroup, which merges MERGE_ITEMS outputs per thread: 512 for keys alone (the
// kernel's time is trips to memory, so large chunks: 2^26 float32 keys in rows of 16 385 0.26 -> 0.23 ms
// against 256), 256 when int64 positions are staged beside the keys (56 KiB of LDS with 512 left two
// workgroups per CU: 0.37 -> 0.44 ms).
__host__ __device__ constexpr int merge_block(bool has_idx) { return has_idx ? 256 : 512; }
__host__ __device__ constexpr int merge_chunk(bool has_idx) { return merge_block(has_idx) * MERGE_ITEMS; }
constexpr int MERGE_CHUNK_MIN = 256 * MERGE_ITEMS;  // the smaller of the two: bounds the grid

// keys / idx: the rows with both halves sorted, [rows][n]; half 0 is [0, h), half 1 [h, n).
// idx holds the final int64 row positions of the elements (those of half 1 already count from h).
// keys_out may be nullptr (index-only sorts), idx / idx_out are nullptr unless HAS_IDX.
template <typename KeyT, int CODEC, bool HAS_IDX>
__global__ __launch_bounds__(merge_block(HAS_IDX)) void merge_halves_kernel(const KeyT* __restrict__ keys,
                                                                    const int64_t* __restrict__ idx,
                                                                    KeyT* __restrict__ keys_out,
                                                                    int64_t* __restrict__ idx_out,
                                                                    uint32_t n,
                                                                    uint32_t h,
                                                                    uint32_t chunks_per_row)
{
  constexpr int MERGE_BLOCK = merge_block(HAS_IDX);
  constexpr int MERGE_CHUNK = merge_chunk(HAS_IDX);
  __shared__ KeyT s_key[MERGE_CHUNK];
  __shared__ int64_t s_idx[HAS_IDX ? MERGE_CHUNK : 1];
  __shared__ uint16_t s_src[HAS_IDX ? MERGE_CHUNK : 1];

  const int tid        = threadIdx.x;
  const uint64_t row   = blockIdx.x / chunks_per_row;
  const uint32_t chunk = blockIdx.x - static_cast<uint32_t>(row * chunks_per_row);
  const KeyT* a        = keys + row * n;  // first half, len_a keys
  const KeyT* b        = a + h;           // second half, len_b keys
  const uint32_t len_a = h, len_b = n - h;
  const uint32_t d0    = chunk * MERGE_CHUNK;
  const uint32_t d1    = (d0 + MERGE_CHUNK < n) ? d0 + MERGE_CHUNK : n;

  auto image = [](KeyT k) { return ordered_bits<CODEC, KeyT>(k); };

  // How many of the first d merged keys come from the first half: the smallest i with
  // !(a[i] <= b[d - 1 - i]).  The whole workgroup looks for it, one candidate per thread and round, for both
  // ends of its chunk in the same rounds (two rounds for halves of up to 65 536 keys: every round
  // is a trip to memory, which is what this kernel's time is made of, hence the large chunks).
  uint32_t lo[2], hi[2];
  const uint32_t dd[2] = {d0, d1};
#pragma unroll
  for (int e = 0; e < 2; ++e) {
    lo[e] = dd[e] > len_b ? dd[e] - len_b : 0u;
    hi[e] = dd[e] < len_a ? dd[e] : len_a;
  }
  while (lo[0] < hi[0] || lo[1] < hi[1]) {  // uniform
    uint32_t step[2];
    int below[2];
#pragma unroll
    for (int e = 0; e < 2; ++e) {
      step[e]             = (hi[e] - lo[e] + MERGE_BLOCK - 1) / MERGE_BLOCK;
      const uint32_t cand = lo[e] + static_cast<uint32_t>(tid) * step[e];
      below[e]            = 0;
      if (cand < hi[e]) {
        below[e] = image(a[cand]) <= image(b[dd[e] - 1 - cand]) ? 1 : 0;
      }
    }
#pragma unroll
    for (int e = 0; e < 2; ++e) {
      const uint32_t k = static_cast<uint32_t>(__syncthreads_count(below[e]));  // candidates before the split: a prefix
      if (lo[e] < hi[e]) {
        if (k == 0) {
          hi[e] = lo[e];
        } else {
          const uint32_t new_hi = lo[e] + k * step[e];
          lo[e]                 = lo[e] + (k - 1) * step[e] + 1;
          hi[e]                 = new_hi < hi[e] ? new_hi : hi[e];
        }
      }
    }
  }
  const uint32_t a0 = lo[0], a1 = lo[1];
  const uint32_t b0 = d0 - a0, b1 = d1 - a1;
  const uint32_t na = a1 - a0, nb = b1 - b0, total = d1 - d0;

  // this chunk's keys of both halves, side by side in LDS (all loads of a thread first, from
  // positions clamped into the chunk, so that none waits for the one before it)
  {
    KeyT v[MERGE_ITEMS];
    int64_t p[HAS_IDX ? MERGE_ITEMS : 1];
#pragma unroll
    for (int k = 0; k < MERGE_ITEMS; ++k) {
      const uint32_t j   = static_cast<uint32_t>(tid) + k * MERGE_BLOCK;
      const uint32_t jj  = j < total ? j : total - 1;
      const uint32_t src = jj < na ? a0 + jj : h + b0 + (jj - na);
      v[k]               = a[src];
      if constexpr (HAS_IDX) {
        p[k] = idx[row * n + src];
      }
    }
#pragma unroll
    for (int k = 0; k < MERGE_ITEMS; ++k) {
      const uint32_t j = static_cast<uint32_t>(tid) + k * MERGE_BLOCK;
      if (j < total) {
        s_key[j] = v[k];
        if constexpr (HAS_IDX) {
          s_idx[j] = p[k];
        }
      }
    }
  }
  __syncthreads();

  // every thread merges MERGE_ITEMS consecutive outputs, from its own split of the chunk
  const uint32_t diag = static_cast<uint32_t>(tid) * MERGE_ITEMS < total ? static_cast<uint32_t>(tid) * MERGE_ITEMS : total;
  uint32_t tlo = diag > nb ? diag - nb : 0u, thi = diag < na ? diag : na;
  while (tlo < thi) {
    const uint32_t mid = (tlo + thi) / 2;
    if (image(s_key[mid]) <= image(s_key[na + (diag - 1 - mid)])) {
      tlo = mid + 1;
    } else {
      thi = mid;
    }
  }
  uint32_t ia = tlo, ib = diag - tlo;
  KeyT out_key[MERGE_ITEMS];
  uint32_t out_src[MERGE_ITEMS];
  // the heads of both runs stay in registers; a step reads only the successor of the key it took
  // (positions past the end of a run are clamped: their keys are read and never taken)
  KeyT head_a = s_key[ia < na ? ia : (na != 0 ? na - 1 : 0)];
  KeyT head_b = s_key[na + (ib < nb ? ib : (nb != 0 ? nb - 1 : 0))];
#pragma unroll
  for (int k = 0; k < MERGE_ITEMS; ++k) {
    out_key[k] = KeyT{};
    out_src[k] = 0;
    if (diag + k < total) {
      const bool take_a = ib >= nb || (ia < na && image(head_a) <= image(head_b));
      out_key[k]        = take_a ? head_a : head_b;
      out_src[k]        = take_a ? ia : na + ib;
      ia += take_a ? 1u : 0u;
      ib += take_a ? 0u : 1u;
      const uint32_t next = take_a ? (ia < na ? ia : ia - 1) : na + (ib < nb ? ib : ib - 1);
      const KeyT v        = s_key[next];
      head_a              = take_a ? v : head_a;
      head_b              = take_a ? head_b : v;
    }
  }
  __syncthreads();  // every thread has read what it needs of s_key
#pragma unroll
  for (int k = 0; k < MERGE_ITEMS; ++k) {
    if (diag + k < total) {
      s_key[diag + k] = out_key[k];
      if constexpr (HAS_IDX) {
        s_src[diag + k] = static_cast<uint16_t>(out_src[k]);
      }
    }
  }
  __syncthreads();
  const uint64_t out_base = row * n + d0;
#pragma unroll
  for (int k = 0; k < MERGE_ITEMS; ++k) {
    const uint32_t j = static_cast<uint32_t>(tid) + k * MERGE_BLOCK;
    if (j < total) {
      if (keys_out != nullptr) {
        keys_out[out_base + j] = s_key[j];
      }
      if constexpr (HAS_IDX) {
        idx_out[out_base + j] = s_idx[s_src[j]];
      }
    }
  }
}

}  // namespace cpn
