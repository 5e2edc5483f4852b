// Rows too long for the per-row kernels: every row is cut into 2^levels pieces of equal length (the
// last one may be shorter), each sorted by the one-workgroup-per-row kernel (a piece fits the LDS of
// a CU), and neighbouring pieces are merged here, level by level, until the row is one run.
// One read and one write of HBM per element and step, against one pass per key byte, per-row
// histograms and tiles that end at every row on the global path.
//
// Stands, for these rows, where the reference runs cub::DeviceSegmentedRadixSort
// (src/cupynumeric/sort/cub_sort.cuh:81-105,153-182).
//
// The merge is stable: of two keys that tie, the one from the first piece of a pair (the lower
// positions of the row) comes first, and inside a piece the stable row sort has kept input order.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "key_codec.h"
#include "radix_common.h"

namespace cpn {

#ifndef CPN_MERGE_ITEMS
#define CPN_MERGE_ITEMS 8
#endif
constexpr int MERGE_ITEMS = CPN_MERGE_ITEMS;
// Threads of a workgroup, which merges MERGE_ITEMS outputs per thread: 512 for keys alone (the
// kernel's time is trips to memory, so large chunks: 2^26 float32 keys in rows of 16 385 0.26 -> 0.23 ms
// against 256), 256 when int64 positions are staged beside the keys (56 KiB of LDS with 512 left two
// workgroups per CU: 0.37 -> 0.44 ms).
__host__ __device__ constexpr int merge_block(bool has_idx) { return has_idx ? 256 : 512; }
__host__ __device__ constexpr int merge_chunk(bool has_idx) { return merge_block(has_idx) * MERGE_ITEMS; }
constexpr int MERGE_CHUNK_MIN = 256 * MERGE_ITEMS;  // the smaller of the two: bounds the grid

// Where a workgroup of the merge starts: blockIdx.x -> row, pair of pieces in the row, chunk of the pair's outputs.
struct MergeChunk {
  uint64_t first;  // of the pair, in keys / idx and in the outputs
  uint32_t len_a, len_b;  // the two pieces (len_b == 0: nothing to merge with)
  uint32_t d0;            // first merged output of the chunk, counted inside the pair
};
__device__ inline MergeChunk merge_chunk_of(
  uint32_t block, uint32_t n, uint32_t piece, uint32_t chunks_per_pair, uint32_t pairs_per_row, uint32_t chunk_len)
{
  uint64_t row;
  uint32_t pair, chunk;
  if (pairs_per_row == 1) {
    row   = block / chunks_per_pair;
    pair  = 0;
    chunk = block - static_cast<uint32_t>(row * chunks_per_pair);
  } else {
    const uint32_t per_row = pairs_per_row * chunks_per_pair;
    row                    = block / per_row;
    const uint32_t rest    = block - static_cast<uint32_t>(row * per_row);
    pair                   = rest / chunks_per_pair;
    chunk                  = rest - pair * chunks_per_pair;
  }
  const uint64_t start = 2ull * pair * piece;  // of this pair in its row; start < n
  const uint32_t left  = n - static_cast<uint32_t>(start);
  MergeChunk c;
  c.first = row * n + start;
  c.len_a = left < piece ? left : piece;
  c.len_b = left - c.len_a < piece ? left - c.len_a : piece;
  c.d0    = chunk * chunk_len;
  return c;
}

// How many of the outputs before a chunk come from the first piece of its pair, for every chunk
// of the merge launch that follows (one thread each): the smallest i with !(a[i] <= b[d0 - 1 - i]).
// Done ahead of the merge because a search inside its workgroups, with one candidate per thread,
// touched a cache line per candidate, four times the lines of the chunk itself.
constexpr int MERGE_SPLIT_BLOCK = 256;
template <typename KeyT, int CODEC>
__global__ __launch_bounds__(MERGE_SPLIT_BLOCK) void merge_split_kernel(const KeyT* __restrict__ keys,
                                                                        uint32_t* __restrict__ splits,
                                                                        uint32_t n,
                                                                        uint32_t piece,
                                                                        uint32_t chunks_per_pair,
                                                                        uint32_t pairs_per_row,
                                                                        uint32_t chunk_len,
                                                                        uint32_t chunks_total)
{
  const uint32_t g = blockIdx.x * MERGE_SPLIT_BLOCK + threadIdx.x;
  if (g >= chunks_total) {
    return;
  }
  const MergeChunk c = merge_chunk_of(g, n, piece, chunks_per_pair, pairs_per_row, chunk_len);
  const uint32_t d   = c.d0 < c.len_a + c.len_b ? c.d0 : c.len_a + c.len_b;  // (chunks past the end of a short pair)
  const KeyT* a      = keys + c.first;
  const KeyT* b      = a + c.len_a;
  uint32_t lo = d > c.len_b ? d - c.len_b : 0u, hi = d < c.len_a ? d : c.len_a;
  while (lo < hi) {
    const uint32_t mid = (lo + hi) / 2;
    if (ordered_bits<CODEC, KeyT>(a[mid]) <= ordered_bits<CODEC, KeyT>(b[d - 1 - mid])) {
      lo = mid + 1;
    } else {
      hi = mid;
    }
  }
  splits[g] = lo;
}

// keys / idx: the rows, [rows][n], every row in sorted pieces of `piece` elements: [0, piece),
// [piece, 2 piece), ... (the last one ends at n).  Pieces 2p and 2p + 1 of a row are merged into
// [2p piece, (2p + 2) piece) of the outputs; a piece without a partner is copied.
// idx holds the final int64 row positions of the elements (they count from the start of the row).
// keys_out may be nullptr (index-only sorts, last level), idx / idx_out are nullptr unless HAS_IDX.
// splits: merge_split_kernel's output for this launch.
// Grid: rows x pairs_per_row x chunks_per_pair workgroups, chunks_per_pair = ceil(2 piece / merge_chunk).
template <typename KeyT, int CODEC, bool HAS_IDX>
__global__ __launch_bounds__(merge_block(HAS_IDX)) void merge_halves_kernel(const KeyT* __restrict__ keys,
                                                                    const int64_t* __restrict__ idx,
                                                                    KeyT* __restrict__ keys_out,
                                                                    int64_t* __restrict__ idx_out,
                                                                    const uint32_t* __restrict__ splits,
                                                                    uint32_t n,
                                                                    uint32_t piece,
                                                                    uint32_t chunks_per_pair,
                                                                    uint32_t pairs_per_row)
{
  constexpr int MERGE_BLOCK = merge_block(HAS_IDX);
  constexpr int MERGE_CHUNK = merge_chunk(HAS_IDX);
  __shared__ KeyT s_key[MERGE_CHUNK];
  __shared__ int64_t s_idx[HAS_IDX ? MERGE_CHUNK : 1];
  __shared__ uint16_t s_src[HAS_IDX ? MERGE_CHUNK : 1];

  const int tid      = threadIdx.x;
  const MergeChunk c = merge_chunk_of(blockIdx.x, n, piece, chunks_per_pair, pairs_per_row, MERGE_CHUNK);
  const uint32_t len_a = c.len_a, len_b = c.len_b, d0 = c.d0;
  const uint32_t h = len_a;  // the second piece starts here
  if (d0 >= len_a + len_b) {
    return;  // (the whole workgroup: the last pair of a row may be short)
  }
  const bool ends      = d0 + MERGE_CHUNK >= len_a + len_b;  // the pair ends in this chunk
  const uint32_t d1    = ends ? len_a + len_b : d0 + MERGE_CHUNK;
  const uint64_t first = c.first;
  const KeyT* a        = keys + first;  // first piece, len_a keys

  auto image = [](KeyT k) { return ordered_bits<CODEC, KeyT>(k); };

  // how many of the outputs before the chunk, and before the next one, come from the first piece
  // (merge_split_kernel; the next chunk of the pair is the next workgroup)
  const uint32_t a0 = splits[blockIdx.x];
  const uint32_t a1 = ends ? len_a : splits[blockIdx.x + 1];
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
        p[k] = idx[first + src];
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
  KeyT head_b = s_key[nb != 0 ? na + (ib < nb ? ib : nb - 1) : 0];
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
  const uint64_t out_base = first + d0;
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
