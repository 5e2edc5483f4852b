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
// Measured on float16 rows, 2^26 keys in all, radix row kernel / this kernel: rows of 3000 0.25 / 0.36 ms,
// 4096 0.23 / 0.30; against the radix kernel's 512-thread shapes of 12 and 16 keys per thread (two workgroups
// per CU): 4097 0.27 / 0.39, 5000 0.22 / 0.28, 6144 0.185 / 0.23, 6145 0.24 / 0.32, 8192 0.18 / 0.20; and
// against its 1024-thread shapes above: 8193 0.42 / 0.38, 12 288 0.35 / 0.21, 16 384 0.33 / 0.19 ms.
// So the counting starts where the 512-thread shapes end (count16_long_rows_kernel); the kernel for rows of
// up to 8192 keys, count16_rows_kernel, runs only when the environment lowers this value.
constexpr uint32_t COUNT16_MIN_ROW = 8193;

// Word of the histogram that holds bin `bin`.  Words are kept in 16-byte chunks and the chunk index is
// XOR-swizzled so that the scan, in which every thread walks 8 consecutive chunks of its own,
// spreads the lanes of a wave over all LDS banks instead of queueing on four of them.
__device__ __forceinline__ uint32_t count16_chunk(uint32_t chunk) { return chunk ^ ((chunk >> 4) & 15u); }
__device__ __forceinline__ uint32_t count16_word(uint32_t bin)
{
  const uint32_t w = bin >> 1;
  return (count16_chunk(w >> 2) << 2) | (w & 3u);
}

// Bin number -> the key's bits (inverse of the ordered image; zeros come back as +0.0, which is what
// a row without -0.0 holds).
template <int CODEC>
__device__ __forceinline__ uint16_t count16_key_of_bin(uint32_t bin)
{
  if constexpr (CODEC == CODEC_UNSIGNED) {
    return static_cast<uint16_t>(bin);
  } else if constexpr (CODEC == CODEC_SIGNED) {
    return static_cast<uint16_t>(bin ^ 0x8000u);
  } else {
    return sign_unflip<uint16_t>(static_cast<uint16_t>(bin));
  }
}

// Sum of the entries of a 16-entry LDS array that lie before `wave`: all sixteen are read at once
// (four 16-byte broadcast reads) instead of one after the other.
__device__ __forceinline__ uint32_t count16_before_wave(const uint32_t* s16, int wave, bool take_max)
{
  const uint4* v = reinterpret_cast<const uint4*>(s16);
  uint32_t e[16];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const uint4 q = v[j];
    e[4 * j] = q.x, e[4 * j + 1] = q.y, e[4 * j + 2] = q.z, e[4 * j + 3] = q.w;
  }
  uint32_t acc = 0;
#pragma unroll
  for (int w = 0; w < 16; ++w) {
    const uint32_t x = (w < wave) ? e[w] : 0u;
    acc              = take_max ? (acc > x ? acc : x) : acc + x;
  }
  return acc;
}

// Rows of up to 8192 keys.  grid <= rows, block = 1024: a workgroup takes rows blockIdx.x,
// blockIdx.x + gridDim.x, ... (the histogram fills most of a CU's LDS, so one workgroup per CU is
// all there is: it stays, loads its next row early and counts it while the current one is written
// out).  Thread t owns elements [8t, 8t+8) of the row on the way in and the same positions of the
// sorted row on the way out.
//
// The sorted row is written out bin by bin rather than key by key: every key stores its bin number
// at the start offset of its bin in a marker row (the same value from every key of the bin), a
// running maximum over the marker row tells each output position its bin (bins ascend with the
// position), and the bin number is mapped back to the key's bits.  No atomic returns a value and
// no key is scattered twice.
template <int CODEC>
__global__ __launch_bounds__(COUNT16_BLOCK) void count16_rows_kernel(const uint16_t* keys_in,
                                                                      uint16_t* keys_out,
                                                                      uint32_t seg,
                                                                      uint32_t rows,
                                                                      uint32_t* status)
{
  static_assert(CODEC == CODEC_UNSIGNED || CODEC == CODEC_SIGNED || CODEC == CODEC_FLOAT, "real 2-byte keys");
  static_assert(COUNT16_BLOCK / WAVE == 16, "count16_before_wave reads sixteen wave totals");
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    *status = 0;  // the workspace's status word: a per-row sort cannot fail on the device
  }
  constexpr int ITEMS = 8;
  constexpr int WAVES = COUNT16_BLOCK / WAVE;
  __shared__ __align__(16) uint32_t s_hist[COUNT16_WORDS];
  __shared__ __align__(16) uint16_t s_mark[COUNT16_BLOCK * ITEMS];
  __shared__ __align__(16) uint32_t s_wsum[WAVES];
  __shared__ __align__(16) uint32_t s_msum[WAVES];
  __shared__ __align__(16) uint32_t s_zsum[WAVES];
  __shared__ __align__(16) uint32_t s_nsum[WAVES];

  const int tid     = threadIdx.x;
  const int lane    = tid & (WAVE - 1);
  const int wave    = tid / WAVE;
  const uint32_t e0 = tid * ITEMS;  // first element of this thread
  // 16-byte accesses reach every row if they reach the first and rows are whole vectors
  const bool vec_in  = ((reinterpret_cast<uintptr_t>(keys_in) & 15u) == 0) && ((seg & 7u) == 0);
  const bool vec_out = ((reinterpret_cast<uintptr_t>(keys_out) & 15u) == 0) && ((seg & 7u) == 0);
  constexpr uint32_t ZERO_BIN = 0x8000u, NAN_BIN = 0xFFFFu;

  auto load_row = [&](uint32_t row) -> uint4 {
    const uint16_t* in = keys_in + static_cast<uint64_t>(row) * seg;
    uint4 v            = make_uint4(0u, 0u, 0u, 0u);
    if (vec_in) {
      if (e0 < seg) {
        v = reinterpret_cast<const uint4*>(in)[tid];
      }
    } else {
      uint16_t k[ITEMS];
#pragma unroll
      for (int i = 0; i < ITEMS; ++i) {
        k[i] = (e0 + i < seg) ? in[e0 + i] : static_cast<uint16_t>(0);
      }
      __builtin_memcpy(&v, k, 16);
    }
    return v;
  };
  // Counts the keys of one row into the (cleared) histogram.  Float keys: also the zeros and NaNs of
  // this thread, for their stable placement, and whether the order inside those two bins shows at
  // all: only if one of them holds different bits; one test covers that and more (any -0.0, any
  // NaN) and costs nothing on ordinary data.
  auto count_row = [&](const uint16_t (&key)[ITEMS], uint32_t& zeros, uint32_t& nans, int& special) {
    zeros = 0, nans = 0, special = 0;
#pragma unroll
    for (int i = 0; i < ITEMS; ++i) {
      if (e0 + i < seg) {
        const uint32_t bin = ordered_bits<CODEC, uint16_t>(key[i]);
        atomicAdd(&s_hist[count16_word(bin)], 1u << (16 * (bin & 1u)));
        if constexpr (CODEC == CODEC_FLOAT) {
          zeros += (bin == ZERO_BIN) ? 1u : 0u;
          nans += (bin == NAN_BIN) ? 1u : 0u;
          special |= (bin != sign_flip<uint16_t>(key[i])) ? 1 : 0;
        }
      }
    }
  };

  uint32_t row = blockIdx.x;
  uint4 loaded = load_row(row);
  {
    uint4* hz = reinterpret_cast<uint4*>(s_hist);
#pragma unroll
    for (int j = 0; j < COUNT16_WORDS / 4 / COUNT16_BLOCK; ++j) {
      hz[tid + j * COUNT16_BLOCK] = make_uint4(0u, 0u, 0u, 0u);
    }
    reinterpret_cast<uint4*>(s_mark)[tid] = make_uint4(0u, 0u, 0u, 0u);
  }
  __syncthreads();

  uint16_t key[ITEMS];
  __builtin_memcpy(key, &loaded, 16);
  uint32_t zeros, nans;
  int special;
  count_row(key, zeros, nans, special);

  for (;;) {
    const int any_special = __syncthreads_or(special);  // (also: every count of this row is in)
    // the next row starts its way here, a few thousand cycles before it is needed
    const uint32_t next_row = row + gridDim.x;
    const bool has_next     = next_row < rows;  // uniform
    if (has_next) {
      loaded = load_row(next_row);
    }

    // ---- exclusive scan of the 65 536 bins: thread t owns bins [64t, 64t+64) = 8 chunks ----
    uint4 q[8];
    uint32_t total = 0;
    {
      const uint4* hv = reinterpret_cast<const uint4*>(s_hist);
#pragma unroll
      for (int k = 0; k < 8; ++k) {
        q[k] = hv[count16_chunk(8u * tid + k)];
        // both halves of every word at once: no sum of halves exceeds the row length
        const uint32_t t = q[k].x + q[k].y + q[k].z + q[k].w;
        total += (t & 0xFFFFu) + (t >> 16);
      }
    }
    const uint32_t incl = wave_inclusive_sum_dpp(total);
    if (lane == WAVE - 1) {
      s_wsum[wave] = incl;
    }
    uint32_t zincl = 0, nincl = 0;
    if constexpr (CODEC == CODEC_FLOAT) {
      if (any_special != 0) {  // uniform: prefix sums of the zeros and NaNs, in row order
        zincl = wave_inclusive_sum_dpp(zeros);
        nincl = wave_inclusive_sum_dpp(nans);
        if (lane == WAVE - 1) {
          s_zsum[wave] = zincl;
          s_nsum[wave] = nincl;
        }
      }
    }
    __syncthreads();
    uint32_t run   = incl - total + count16_before_wave(s_wsum, wave, false);
    uint32_t zrank = zincl - zeros, nrank = nincl - nans;
    if constexpr (CODEC == CODEC_FLOAT) {
      if (any_special != 0) {
        zrank += count16_before_wave(s_zsum, wave, false);
        nrank += count16_before_wave(s_nsum, wave, false);
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

    // ---- every key marks the start of its bin ----
    uint32_t zstart = 0, nstart = 0;
#pragma unroll
    for (int i = 0; i < ITEMS; ++i) {
      if (e0 + i < seg) {
        const uint32_t bin   = ordered_bits<CODEC, uint16_t>(key[i]);
        const uint32_t start = (s_hist[count16_word(bin)] >> (16 * (bin & 1u))) & 0xFFFFu;
        s_mark[start]        = static_cast<uint16_t>(bin);
        if constexpr (CODEC == CODEC_FLOAT) {
          zstart = (bin == ZERO_BIN) ? start : zstart;
          nstart = (bin == NAN_BIN) ? start : nstart;
        }
      }
    }
    __syncthreads();  // every offset has been looked up, every marker is set

    // the next row finds an empty histogram: whoever wrote offsets clears them (the counts all lie there)
    if (total != 0) {
      uint4* hv = reinterpret_cast<uint4*>(s_hist);
#pragma unroll
      for (int k = 0; k < 8; ++k) {
        hv[count16_chunk(8u * tid + k)] = make_uint4(0u, 0u, 0u, 0u);
      }
    }

    // ---- the bin of every output position: running maximum of the markers ----
    uint32_t m[ITEMS];
    {
      const uint4 v       = reinterpret_cast<const uint4*>(s_mark)[tid];
      const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        m[2 * j]     = w[j] & 0xFFFFu;
        m[2 * j + 1] = w[j] >> 16;
      }
      reinterpret_cast<uint4*>(s_mark)[tid] = make_uint4(0u, 0u, 0u, 0u);  // (only this thread reads these markers)
    }
#pragma unroll
    for (int i = 1; i < ITEMS; ++i) {
      m[i] = max(m[i], m[i - 1]);
    }
    const uint32_t mincl = wave_inclusive_max_dpp(m[ITEMS - 1]);
    if (lane == WAVE - 1) {
      s_msum[wave] = mincl;
    }
    // (the maximum over the lanes before this one: a one-lane shift of the inclusive scan)
    uint32_t carry = static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(mincl), 0x138 /* wave_shr:1 */, 0xF, 0xF, true));
    __syncthreads();  // the histogram is clear, the markers have been read
    carry = max(carry, count16_before_wave(s_msum, wave, true));

    // The next row is counted before this one is written out: its atomics drain while the bins of
    // this row are turned back into keys.
    uint16_t key_next[ITEMS];
    uint32_t zeros_next = 0, nans_next = 0;
    int special_next    = 0;
    if (has_next) {
      __builtin_memcpy(key_next, &loaded, 16);
      count_row(key_next, zeros_next, nans_next, special_next);
    }

    uint32_t packed[ITEMS / 2];
#pragma unroll
    for (int i = 0; i < ITEMS; ++i) {
      const uint32_t raw = count16_key_of_bin<CODEC>(max(m[i], carry));
      packed[i / 2]      = (i % 2 == 0) ? raw : (packed[i / 2] | (raw << 16));
    }
    const uint4 mine = make_uint4(packed[0], packed[1], packed[2], packed[3]);
    uint16_t* out    = keys_out + static_cast<uint64_t>(row) * seg;
    if (any_special == 0 && vec_out) {  // uniform
      if (e0 < seg) {
        reinterpret_cast<uint4*>(out)[tid] = mine;
      }
    } else {
      // rows with a -0.0 or a NaN, and rows that 16-byte stores cannot reach: through the marker row
      reinterpret_cast<uint4*>(s_mark)[tid] = mine;
      __syncthreads();
      if constexpr (CODEC == CODEC_FLOAT) {
        if (any_special != 0) {
          // zeros and NaNs keep their own bits, in input order
#pragma unroll
          for (int i = 0; i < ITEMS; ++i) {
            if (e0 + i < seg) {
              const uint32_t bin = ordered_bits<CODEC_FLOAT, uint16_t>(key[i]);
              if (bin == ZERO_BIN) {
                s_mark[zstart + zrank++] = key[i];
              } else if (bin == NAN_BIN) {
                s_mark[nstart + nrank++] = key[i];
              }
            }
          }
          __syncthreads();
        }
      }
      if (vec_out) {
        if (e0 < seg) {
          reinterpret_cast<uint4*>(out)[tid] = reinterpret_cast<const uint4*>(s_mark)[tid];
        }
      } else {
        for (uint32_t o = tid; o < seg; o += COUNT16_BLOCK) {
          out[o] = s_mark[o];
        }
      }
      __syncthreads();
      reinterpret_cast<uint4*>(s_mark)[tid] = make_uint4(0u, 0u, 0u, 0u);
    }
    if (!has_next) {
      break;
    }
    row = next_row;
#pragma unroll
    for (int i = 0; i < ITEMS; ++i) {
      key[i] = key_next[i];
    }
    zeros = zeros_next, nans = nans_next, special = special_next;
  }
}

// Rows of 8193 to 16 384 keys (ITEMS = 16), of up to 32 768 (ITEMS = 32) and of up to 57 344 (ITEMS = 56).  grid = rows, block = 1024,
// thread t owns elements [ITEMS t, ITEMS (t + 1)).
// No LDS is left for a marker row here: every key takes its offset from an atomic on the scanned
// histogram and is staged in the histogram's memory once that is no longer needed (65 536 bins of 16
// bits are room for 65 536 keys; a bin counts up to 65 535, more than the longest row).
template <int CODEC, int ITEMS>
__global__ __launch_bounds__(COUNT16_BLOCK) void count16_long_rows_kernel(const uint16_t* keys_in,
                                                                           uint16_t* keys_out,
                                                                           uint32_t seg,
                                                                           uint32_t* status)
{
  static_assert(CODEC == CODEC_UNSIGNED || CODEC == CODEC_SIGNED || CODEC == CODEC_FLOAT, "real 2-byte keys");
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    *status = 0;  // the workspace's status word: a per-row sort cannot fail on the device
  }
  static_assert(ITEMS % 8 == 0 && COUNT16_BLOCK * ITEMS < 65536, "whole 16-byte loads; counts and offsets fit 16 bits");
  constexpr int WAVES = COUNT16_BLOCK / WAVE;
  __shared__ __align__(16) uint32_t s_hist[COUNT16_WORDS];
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
  }
  __syncthreads();

  // ---- count.  Float keys: the zeros and the NaNs of this thread, for their stable placement ----
  constexpr uint32_t ZERO_BIN = 0x8000u, NAN_BIN = 0xFFFFu;
  uint32_t zeros = 0, nans = 0;
  int special = 0;
#pragma unroll
  for (int i = 0; i < ITEMS; ++i) {
    if (e0 + i < seg) {
      const uint32_t bin = ordered_bits<CODEC, uint16_t>(key[i]);
      atomicAdd(&s_hist[count16_word(bin)], 1u << (16 * (bin & 1u)));
      if constexpr (CODEC == CODEC_FLOAT) {
        zeros += (bin == ZERO_BIN) ? 1u : 0u;
        nans += (bin == NAN_BIN) ? 1u : 0u;
        special |= (bin != sign_flip<uint16_t>(key[i])) ? 1 : 0;  // any -0.0, any NaN
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
      const uint32_t t = q[k].x + q[k].y + q[k].z + q[k].w;
      total += (t & 0xFFFFu) + (t >> 16);
    }
  }
  const uint32_t incl = wave_inclusive_scan(total, lane);
  if (lane == WAVE - 1) {
    s_wsum[wave] = incl;
  }
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

  uint16_t* out      = keys_out + base;
  const bool vec_out = ((reinterpret_cast<uintptr_t>(out) & 15u) == 0) && ((seg & 7u) == 0);  // uniform
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

}  // namespace cpn
