// Building blocks shared by the global (onesweep) and the per-row (LDS) radix sorts:
// wave64 match-any ranking, the per-tile digit scan, and small helpers.
//
// Replaces what the reference gets from cub's block/warp radix-rank primitives behind
// cub::DeviceRadixSort / DeviceSegmentedRadixSort (src/cupynumeric/sort/cub_sort.cuh:60-182).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "key_codec.h"

namespace cpn {

constexpr int RADIX_BITS = 8;
constexpr int RADIX      = 1 << RADIX_BITS;
constexpr int WAVE       = 64;

__device__ __forceinline__ uint32_t lanes_below(uint64_t mask)
{
  return __builtin_amdgcn_mbcnt_hi(static_cast<uint32_t>(mask >> 32),
                                   __builtin_amdgcn_mbcnt_lo(static_cast<uint32_t>(mask), 0u));
}

// Stable rank of one key per lane inside a wave, keys ordered by lane id.
//
//   digit   8-bit digit of this lane's key
//   valid   lane holds a real key
//   wctr    this wave's 256 running digit counters in LDS (count of that digit in the
//           wave's earlier rounds)
//
// Returns the number of keys with the same digit that precede this key in the wave
// (earlier rounds + lower lanes of this round) and advances the counter.  Eight ballots
// build the mask of lanes holding the same digit: for every digit bit, a lane accumulates
// the lanes whose bit differs from its own (ballot XOR own bit broadcast over 32 bits).
// The highest lane of each group updates the counter after every member has read it (LDS
// operations of one wave execute in order).
__device__ __forceinline__ uint32_t wave_match_rank(uint32_t digit, bool valid, uint32_t* wctr)
{
  const uint64_t vmask = __builtin_amdgcn_ballot_w64(valid);
  uint32_t mis_lo = 0, mis_hi = 0;
#pragma unroll
  for (int b = 0; b < RADIX_BITS; ++b) {
    int32_t own = __builtin_amdgcn_sbfe(static_cast<int32_t>(digit), b, 1);  // 0 or -1
    asm volatile("" : "+v"(own));  // keep the compare on `own` (one v_cmp) instead of a re-derived bit test
    const uint64_t bal = __builtin_amdgcn_ballot_w64(own != 0);
    // mis |= bal ^ own, one three-input bit operation per half (truth table 0xF6 = a | (b ^ c))
    mis_lo = __builtin_amdgcn_bitop3_b32(mis_lo, static_cast<uint32_t>(bal), static_cast<uint32_t>(own), 0xF6);
    mis_hi = __builtin_amdgcn_bitop3_b32(mis_hi, static_cast<uint32_t>(bal >> 32), static_cast<uint32_t>(own), 0xF6);
  }
  const uint32_t peers_lo = static_cast<uint32_t>(vmask) & ~mis_lo;
  const uint32_t peers_hi = static_cast<uint32_t>(vmask >> 32) & ~mis_hi;
  const uint32_t lower    = __builtin_amdgcn_mbcnt_hi(peers_hi, __builtin_amdgcn_mbcnt_lo(peers_lo, 0u));
  const uint32_t total    = static_cast<uint32_t>(__builtin_popcount(peers_lo) + __builtin_popcount(peers_hi));
  const uint32_t old      = wctr[digit];
  __builtin_amdgcn_wave_barrier();
  if (valid && lower + 1 == total) {
    wctr[digit] = old + total;
  }
  __builtin_amdgcn_wave_barrier();
  return old + lower;
}

// Inclusive scan of one 32-bit value per lane across a wave.
__device__ __forceinline__ uint32_t wave_inclusive_scan(uint32_t v, int lane)
{
#pragma unroll
  for (int delta = 1; delta < WAVE; delta <<= 1) {
    const uint32_t t = __shfl_up(v, delta, WAVE);
    if (lane >= delta) {
      v += t;
    }
  }
  return v;
}

// Inclusive scans across a wave through DPP lane moves (no LDS traffic, a few cycles per step, where
// a shuffle goes through the LDS crossbar): four shifts inside each row of 16 lanes, then the last
// lane of row 0 is added to row 1 and that of row 2 to row 3, then lane 31 to rows 2 and 3.  Lanes
// without a source read 0, the identity of both operations (values are unsigned).
template <bool MAX>
__device__ __forceinline__ uint32_t wave_inclusive_scan_dpp_impl(uint32_t v)
{
  auto combine = [](uint32_t a, uint32_t b) -> uint32_t { return MAX ? (a > b ? a : b) : a + b; };
  const int x  = static_cast<int>(v);
  // row_shr:1 = 0x111, row_shr:2 = 0x112, row_shr:4 = 0x114, row_shr:8 = 0x118, row_bcast:15 = 0x142, row_bcast:31 = 0x143
  uint32_t t = static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, x, 0x111, 0xF, 0xF, true));
  v          = combine(v, t);
  t          = static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), 0x112, 0xF, 0xF, true));
  v          = combine(v, t);
  t          = static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), 0x114, 0xF, 0xF, true));
  v          = combine(v, t);
  t          = static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), 0x118, 0xF, 0xF, true));
  v          = combine(v, t);
  t          = static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), 0x142, 0xA, 0xF, false));
  v          = combine(v, t);
  t          = static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), 0x143, 0xC, 0xF, false));
  v          = combine(v, t);
  return v;
}
__device__ __forceinline__ uint32_t wave_inclusive_sum_dpp(uint32_t v) { return wave_inclusive_scan_dpp_impl<false>(v); }
__device__ __forceinline__ uint32_t wave_inclusive_max_dpp(uint32_t v) { return wave_inclusive_scan_dpp_impl<true>(v); }

// AND / OR of one 32-bit value per lane over the whole wave, through the same DPP steps (lanes
// without a source keep the identity); the result is read from the last lane and is uniform.
template <bool IS_AND>
__device__ __forceinline__ uint32_t wave_reduce_bits_dpp(uint32_t v)
{
  constexpr int ID = IS_AND ? -1 : 0;
  auto combine     = [](uint32_t a, uint32_t b) -> uint32_t { return IS_AND ? (a & b) : (a | b); };
  uint32_t t       = static_cast<uint32_t>(__builtin_amdgcn_update_dpp(ID, static_cast<int>(v), 0x111, 0xF, 0xF, false));
  v                = combine(v, t);
  t                = static_cast<uint32_t>(__builtin_amdgcn_update_dpp(ID, static_cast<int>(v), 0x112, 0xF, 0xF, false));
  v                = combine(v, t);
  t                = static_cast<uint32_t>(__builtin_amdgcn_update_dpp(ID, static_cast<int>(v), 0x114, 0xF, 0xF, false));
  v                = combine(v, t);
  t                = static_cast<uint32_t>(__builtin_amdgcn_update_dpp(ID, static_cast<int>(v), 0x118, 0xF, 0xF, false));
  v                = combine(v, t);
  t                = static_cast<uint32_t>(__builtin_amdgcn_update_dpp(ID, static_cast<int>(v), 0x142, 0xA, 0xF, false));
  v                = combine(v, t);
  t                = static_cast<uint32_t>(__builtin_amdgcn_update_dpp(ID, static_cast<int>(v), 0x143, 0xC, 0xF, false));
  v                = combine(v, t);
  return static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(v), WAVE - 1));
}
// (any unsigned type of 4 or 8 bytes; the halves of a 64-bit value are reduced on their own)
template <bool IS_AND, typename T>
__device__ __forceinline__ T wave_reduce_bits(T v)
{
  static_assert(sizeof(T) == 4 || sizeof(T) == 8, "32- or 64-bit values");
  if constexpr (sizeof(T) == 4) {
    return static_cast<T>(wave_reduce_bits_dpp<IS_AND>(static_cast<uint32_t>(v)));
  } else {
    const uint32_t hi = wave_reduce_bits_dpp<IS_AND>(static_cast<uint32_t>(static_cast<uint64_t>(v) >> 32));
    const uint32_t lo = wave_reduce_bits_dpp<IS_AND>(static_cast<uint32_t>(v));
    return static_cast<T>((static_cast<uint64_t>(hi) << 32) | lo);
  }
}
template <typename T>
__device__ __forceinline__ T wave_reduce_and_dpp(T v)
{
  return wave_reduce_bits<true, T>(v);
}
template <typename T>
__device__ __forceinline__ T wave_reduce_or_dpp(T v)
{
  return wave_reduce_bits<false, T>(v);
}

// How the 256 digits of a tile are spread over the threads that scan them.
template <int BLOCK>
struct DigitThreads {
  static_assert(BLOCK % WAVE == 0 && BLOCK >= WAVE, "block must be whole waves");
  static constexpr int PER_THREAD = (BLOCK >= RADIX) ? 1 : RADIX / BLOCK;  // digits per scanning thread
  static constexpr int THREADS    = RADIX / PER_THREAD;                      // scanning threads
  static constexpr int WAVES      = THREADS / WAVE;
};

}  // namespace cpn
