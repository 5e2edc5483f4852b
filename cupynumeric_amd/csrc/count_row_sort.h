// Per-row counting sort for 2-byte keys, values only: a row of such keys takes at most 65 536
// different values, so one workgroup counts them in a 65 536-bin histogram in LDS (16-bit counters,
// two to a word, 128 KiB of the CU's 160), scans the histogram and places every key at the
// running offset of its bin.  The work per key is two LDS atomics and a few instructions instead
// of the two ranked 8-bit passes of the radix kernel (sixteen ballots per key).
//
// Replaces, for these rows, cub::DeviceSegmentedRadixSort::SortKeys
// (src/cupynumeric/sort/cub_sort.cuh:81-105).
//
// Why the result is the stable sort although the offset of a key inside its bin comes from an
// atomic counter: keys of one bin are the same bits, so their order does not show.  The two bins
// for which that is not so, the zeros of floats (-0.0 and +0.0 tie) and the NaNs (every sign and
// payload ties), are placed in input order through a prefix sum over the row instead.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "radix_common.h"

namespace cpn {

constexpr int COUNT16_BLOCK = 1024;
constexpr int COUNT16_WORDS = 32768;  // 65 536 bins, two 16-bit counters per word
// Shortest row given to this kernel: below it the fixed cost of clearing and scanning 65 536 bins
// outweighs the cheaper ranking (CPN_SORT_COUNT16_MIN_ROW in the environment overrides it).
constexpr uint32_t COUNT16_MIN_ROW = 2048;

// Word of the histogram that holds bin `bin`.  Words are kept in 16-byte chunks and the chunk index is
// XOR-swizzled so that the scan, in which every thread walks 8 consecutive chunks of its own,
// spreads the lanes of a wave over all LDS banks instead of queueing on four of them.
__device__ __forceinline__ uint32_t count16_chunk(uint32_t chunk) { return chunk ^ ((chunk >> 4) & 15u); }
__device__ __forceinline__ uint32_t count16_word(uint32_t bin)
{
  const uint32_t w = bin >> 1;
  return (count16_chunk(w >> 2) << 2) | (w & 3u);
}

// grid = rows, block = 1024.  Thread t owns elements [t*ITEMS, (t+1)*ITEMS) of its row.
//
// ITEMS == 8 (rows of up to 8192 keys): the sorted row is written out bin by bin.  Every key stores
// its bin number at the start offset of the bin in a 16 KiB marker row (same value from every key
// of the bin), a running maximum over the marker row then tells each output position its bin, and
// the bin number is mapped back to the key's bits: no atomic returns a value and nothing is
// scattered twice.  ITEMS == 16 (up to 16 384 keys) has no LDS left for the marker row; there every
// key takes its offset from an atomic on the scanned histogram and is staged in the histogram's
// memory once that is no longer needed.
template <int CODEC, int ITEMS>
__global__ __launch_bounds__(COUNT16_BLOCK) void count16_row_sort_kernel(const uint16_t* keys_in,
                                                                         uint16_t* keys_out,
                                                                         uint32_t seg,
                                                                         uint32_t* status)
{
  static_assert(ITEMS == 8 || ITEMS == 16, "a thread's keys are one or two 16-byte vectors");
  static_assert(CODEC == CODEC_UNSIGNED || CODEC == CODEC_SIGNED || CODEC == CODEC_FLOAT, "real 2-byte keys");
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    *status = 0;  // the workspace's status word: a per-row sort cannot fail on the device
  }
  constexpr int WAVES    = COUNT16_BLOCK / WAVE;
  constexpr bool MARKERS = (ITEMS == 8);
  __shared__ __align__(16) uint32_t s_hist[COUNT16_WORDS];
  __shared__ __align__(16) uint16_t s_mark[MARKERS ? COUNT16_BLOCK * ITEMS : 8];
  __shared__ uint32_t s_wsum[WAVES];
  __shared__ uint32_t s_zsum[WAVES];
  __shared__ uint32_t s_nsum[WAVES];

  const int tid       = threadIdx.x;
  const int lane      = tid & (WAVE - 1);
  const int wave      = tid / WAVE;
  const uint64_t base = static_cast<uint64_t>(blockIdx.x) * seg;
  const uint32_t e0   = tid * ITEMS;  // first element of this thread

  // ---- load (issued before the histogram is cleared, so that the clearing hides its latency) ----
  const uint16_t* in = keys_in + base;
  const bool vec_in  = ((reinterpret_cast<uintptr_t>(in) & 15u) == 0) && (e0 + ITEMS <= seg);
  uint16_t key[ITEMS];
  if (vec_in) {
    const uint4* vp = reinterpret_cast<const uint4*>(in + e0);
#pragma unroll
    for (int v = 0; v < ITEMS / 8; ++v) {
      const uint4 q = vp[v];
      __builtin_memcpy(key + 8 * v, &q, 16);
    }
  } else {
#pragma unroll
    for (int i = 0; i < ITEMS; ++i) {
      key[i] = (e0 + i < seg) ? in[e0 + i] : static_cast<uint16_t>(0);
    }
  }

  {
    uint4* hz = reinterpret_cast<uint4*>(s_hist);
#pragma unroll
    for (int j = 0; j < COUNT16_WORDS / 4 / COUNT16_BLOCK; ++j) {
      hz[tid + j * COUNT16_BLOCK] = make_uint4(0u, 0u, 0u, 0u);
    }
    if constexpr (MARKERS) {
      reinterpret_cast<uint4*>(s_mark)[tid] = make_uint4(0u, 0u, 0u, 0u);
    }
  }
  __syncthreads();

  // ---- count.  Float keys: the zeros and the NaNs of this thread, for their stable placement ----
  constexpr uint32_t ZERO_BIN = 0x8000u, NAN_BIN = 0xFFFFu;
  uint32_t zeros = 0, nans = 0;
#pragma unroll
  for (int i = 0; i < ITEMS; ++i) {
    if (e0 + i < seg) {
      const uint32_t bin = ordered_bits<CODEC, uint16_t>(key[i]);
      atomicAdd(&s_hist[count16_word(bin)], 1u << (16 * (bin & 1u)));
      if constexpr (CODEC == CODEC_FLOAT) {
        zeros += (bin == ZERO_BIN) ? 1u : 0u;
        nans += (bin == NAN_BIN) ? 1u : 0u;
      }
    }
  }
  // Does the order inside the two special bins show?  Only if one of them holds different bits:
  // a -0.0 beside a +0.0, or NaNs of different payloads; a single test covers both and more
  // (any -0.0, any NaN), which costs nothing on ordinary data.
  int special = 0;
  if constexpr (CODEC == CODEC_FLOAT) {
#pragma unroll
    for (int i = 0; i < ITEMS; ++i) {
      if (e0 + i < seg) {
        special |= (ordered_bits<CODEC_FLOAT, uint16_t>(key[i]) != sign_flip<uint16_t>(key[i])) ? 1 : 0;
      }
    }
  }
  const int any_special = __syncthreads_or(special);  // (also: every count is in)

  // ---- exclusive scan of the 65 536 bins: thread t owns bins [64t, 64t+64) = 8 chunks ----
  uint4 q[8];
  uint32_t total = 0;
  {
    const uint4* hv = reinterpret_cast<const uint4*>(s_hist);
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      q[k] = hv[count16_chunk(8u * tid + k)];
      // both halves of every word: no half exceeds the row length, so the sum of the words' halves
      // is the sum of the words with the high halves shifted down
      const uint32_t s = q[k].x + q[k].y + q[k].z + q[k].w;
      total += (s & 0xFFFFu) + (s >> 16);
    }
  }
  uint32_t incl = wave_inclusive_scan(total, lane);
  if (lane == WAVE - 1) {
    s_wsum[wave] = incl;
  }
  // stable placement of the special bins: prefix sums of this thread's zeros and NaNs
  uint32_t zincl = 0, nincl = 0;
  if constexpr (CODEC == CODEC_FLOAT) {
    if (any_special != 0) {  // uniform
      zincl = wave_inclusive_scan(zeros, lane);
      nincl = wave_inclusive_scan(nans, lane);
      if (lane == WAVE - 1) {
        s_zsum[wave] = zincl;
        s_nsum[wave] = nincl;
      }
    }
  }
  __syncthreads();
  uint32_t run = incl - total;
  for (int w = 0; w < wave; ++w) {
    run += s_wsum[w];
  }
  uint32_t zrank = zincl - zeros, nrank = nincl - nans;  // specials before this thread's, in row order
  if constexpr (CODEC == CODEC_FLOAT) {
    if (any_special != 0) {
      for (int w = 0; w < wave; ++w) {
        zrank += s_zsum[w];
        nrank += s_nsum[w];
      }
    }
  }
  if (total != 0) {  // (offsets of empty bins are never looked up)
    uint4* hv = reinterpret_cast<uint4*>(s_hist);
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      uint32_t w[4] = {q[k].x, q[k].y, q[k].z, q[k].w};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const uint32_t lo = run;
        run += w[j] & 0xFFFFu;
        const uint32_t hi = run;
        run += w[j] >> 16;
        w[j] = lo | (hi << 16);
      }
      hv[count16_chunk(8u * tid + k)] = make_uint4(w[0], w[1], w[2], w[3]);
    }
  }
  __syncthreads();

  uint16_t* out      = keys_out + base;
  const bool vec_out = ((reinterpret_cast<uintptr_t>(out) & 15u) == 0) && ((seg & 7u) == 0);  // uniform

  if constexpr (MARKERS) {
    // ---- every key marks the start of its bin ----
#pragma unroll
    for (int i = 0; i < ITEMS; ++i) {
      if (e0 + i < seg) {
        const uint32_t bin   = ordered_bits<CODEC, uint16_t>(key[i]);
        const uint32_t start = (s_hist[count16_word(bin)] >> (16 * (bin & 1u))) & 0xFFFFu;
        s_mark[start]        = static_cast<uint16_t>(bin);
      }
    }
    __syncthreads();
    // ---- the bin of every output position: running maximum of the markers (bins ascend with the
    //      position, so the maximum so far is the last marker at or before the position) ----
    uint32_t m[ITEMS];
    {
      const uint4 v = reinterpret_cast<const uint4*>(s_mark)[tid];
      const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        m[2 * j]     = w[j] & 0xFFFFu;
        m[2 * j + 1] = w[j] >> 16;
      }
    }
#pragma unroll
    for (int i = 1; i < ITEMS; ++i) {
      m[i] = max(m[i], m[i - 1]);
    }
    uint32_t mincl = m[ITEMS - 1];
#pragma unroll
    for (int delta = 1; delta < WAVE; delta <<= 1) {
      const uint32_t t = __shfl_up(mincl, delta, WAVE);
      if (lane >= delta) {
        mincl = max(mincl, t);
      }
    }
    if (lane == WAVE - 1) {
      s_wsum[wave] = mincl;
    }
    uint32_t carry = __shfl_up(mincl, 1, WAVE);
    if (lane == 0) {
      carry = 0;
    }
    __syncthreads();  // (every marker has been read: s_mark may be written again)
    for (int w = 0; w < wave; ++w) {
      carry = max(carry, s_wsum[w]);
    }
    uint32_t packed[ITEMS / 2];
#pragma unroll
    for (int i = 0; i < ITEMS; ++i) {
      const uint16_t bin = static_cast<uint16_t>(max(m[i], carry));
      uint16_t raw;
      if constexpr (CODEC == CODEC_UNSIGNED) {
        raw = bin;
      } else if constexpr (CODEC == CODEC_SIGNED) {
        raw = static_cast<uint16_t>(bin ^ 0x8000u);
      } else {
        raw = sign_unflip<uint16_t>(bin);  // (+0.0 for the zeros: the only zeros of a row without specials)
      }
      packed[i / 2] = (i % 2 == 0) ? raw : (packed[i / 2] | (static_cast<uint32_t>(raw) << 16));
    }
    const uint4 mine = make_uint4(packed[0], packed[1], packed[2], packed[3]);
    if (any_special == 0 && vec_out) {  // uniform
      if (e0 < seg) {
        reinterpret_cast<uint4*>(out)[tid] = mine;
      }
      return;
    }
    // rows with a -0.0 or a NaN, and rows that 16-byte stores cannot reach: through the marker row
    reinterpret_cast<uint4*>(s_mark)[tid] = mine;
    if constexpr (CODEC == CODEC_FLOAT) {
      if (any_special != 0) {
        __syncthreads();
        // zeros and NaNs keep their own bits, in input order
#pragma unroll
        for (int i = 0; i < ITEMS; ++i) {
          if (e0 + i < seg) {
            const uint32_t bin = ordered_bits<CODEC_FLOAT, uint16_t>(key[i]);
            if (bin == ZERO_BIN || bin == NAN_BIN) {
              const uint32_t start = (s_hist[count16_word(bin)] >> (16 * (bin & 1u))) & 0xFFFFu;
              s_mark[start + ((bin == ZERO_BIN) ? zrank++ : nrank++)] = key[i];
            }
          }
        }
      }
    }
    __syncthreads();
    if (vec_out) {
      if (e0 < seg) {
        reinterpret_cast<uint4*>(out)[tid] = reinterpret_cast<const uint4*>(s_mark)[tid];
      }
    } else {
      for (uint32_t o = tid; o < seg; o += COUNT16_BLOCK) {
        out[o] = s_mark[o];
      }
    }
  } else {
    // ---- place: the running offset of the key's bin (an atomic on its half of the word: the low
    //      half never carries into the high one, it stays below the row length) ----
    uint32_t pos[ITEMS];
#pragma unroll
    for (int i = 0; i < ITEMS; ++i) {
      pos[i] = 0;
      if (e0 + i < seg) {
        const uint32_t bin   = ordered_bits<CODEC, uint16_t>(key[i]);
        const uint32_t shift = 16 * (bin & 1u);
        bool placed          = false;
        if constexpr (CODEC == CODEC_FLOAT) {
          if (any_special != 0 && (bin == ZERO_BIN || bin == NAN_BIN)) {
            // nothing adds to these two bins: the word's half still holds the start of the bin
            const uint32_t start = (s_hist[count16_word(bin)] >> shift) & 0xFFFFu;
            pos[i]               = start + ((bin == ZERO_BIN) ? zrank++ : nrank++);
            placed               = true;
          }
        }
        if (!placed) {
          pos[i] = (atomicAdd(&s_hist[count16_word(bin)], 1u << shift) >> shift) & 0xFFFFu;
        }
      }
    }
    __syncthreads();  // the histogram is no longer needed: its memory now stages the sorted row

    uint16_t* stage = reinterpret_cast<uint16_t*>(s_hist);
#pragma unroll
    for (int i = 0; i < ITEMS; ++i) {
      if (e0 + i < seg) {
        stage[pos[i]] = key[i];
      }
    }
    __syncthreads();

    if (vec_out) {
      const uint4* sv = reinterpret_cast<const uint4*>(stage);
      uint4* ov       = reinterpret_cast<uint4*>(out);
      for (uint32_t c = tid; c < seg / 8; c += COUNT16_BLOCK) {
        ov[c] = sv[c];
      }
    } else {
      for (uint32_t o = tid; o < seg; o += COUNT16_BLOCK) {
        out[o] = stage[o];
      }
    }
  }
}

}  // namespace cpn
