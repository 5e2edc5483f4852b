// Virtual digits: fewer radix passes for keys whose bytes take few distinct values.
//
// The histogram sweep tells, for every byte position of the ordered key, which of the 256
// values occur at all.  A position with d distinct values carries ceil(log2 d) bits of
// information: its bytes can be replaced by their rank among the occurring values (an
// order-preserving code of that many bits).  Neighbouring positions whose codes fit into 8
// bits together are sorted in ONE pass on the concatenation of their codes, which orders the
// keys exactly as the separate byte passes would.  Keys drawn from a small set of arbitrary
// 64-bit values (16 distinct int64 keys: 4 bits per byte) sort in 4 passes instead of 8; keys
// whose bytes are all busy gain nothing and keep the ordinary passes.
//
// The reference's cub::DeviceRadixSort (src/cupynumeric/sort/cub_sort.cuh:60-182) always runs
// sizeof(key) passes of 8 bits.
//
// Everything is decided on the device after the histogram sweep (vplan_kernel); when the plan
// is enabled a second sweep (vhist_kernel) builds the histograms of the virtual digits and the
// scatter passes extract them through per-position lookup tables held in LDS.  Single rows of
// real keys of at most 8 bytes only.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "radix_common.h"

namespace cpn {

constexpr int VIRT_MAX_POSITIONS = 8;  // byte positions of a key (keys of at most 8 bytes)

struct VirtGroup {
  uint32_t count;                      // byte positions forming this virtual digit
  uint32_t pos[VIRT_MAX_POSITIONS];    // which bytes of the ordered key
  uint32_t shift[VIRT_MAX_POSITIONS];  // where each code goes inside the digit
};

struct VirtPlan {
  uint32_t enabled;   // 0: ordinary byte passes
  uint32_t n_groups;  // virtual passes, one per group, least significant first
  VirtGroup group[VIRT_MAX_POSITIONS];
  uint8_t lut[VIRT_MAX_POSITIONS][RADIX];  // per byte position: byte value -> code
};
constexpr uint64_t VIRT_PLAN_BYTES = 4096;
static_assert(sizeof(VirtPlan) <= VIRT_PLAN_BYTES, "plan does not fit its workspace slot");

// One workgroup of 256 threads.  `hist` holds the exclusive-scanned byte histograms of the one
// row ([pass][256]); `varying[p]` says whether position p differs between keys at all.
// When virtual digits save enough passes to pay for themselves: writes the plan, clears hist[g][*] for the
// groups (vhist_kernel accumulates there) and resets varying (the second scan raises it again
// for the groups).  Otherwise leaves everything alone with enabled == 0.
template <typename OffT>
__global__ __launch_bounds__(RADIX) void vplan_kernel(OffT* __restrict__ hist,
                                                       uint32_t* __restrict__ varying,
                                                       VirtPlan* __restrict__ plan,
                                                       uint64_t seg,
                                                       uint32_t passes)
{
  __shared__ uint32_t s_wcount[RADIX / WAVE];
  __shared__ uint32_t s_distinct[VIRT_MAX_POSITIONS];
  __shared__ uint32_t s_enabled, s_groups;
  const int tid  = threadIdx.x;
  const int lane = tid & (WAVE - 1);
  const int wave = tid / WAVE;

  for (uint32_t p = 0; p < passes; ++p) {
    const OffT* h    = hist + static_cast<uint64_t>(p) * RADIX;
    const OffT cur   = h[tid];
    const OffT next  = (tid == RADIX - 1) ? static_cast<OffT>(seg) : h[tid + 1];
    const bool there = (next != cur);  // value `tid` occurs at byte position p
    const uint64_t b = __builtin_amdgcn_ballot_w64(there);
    if (lane == 0) {
      s_wcount[wave] = static_cast<uint32_t>(__builtin_popcountll(b));
    }
    __syncthreads();
    uint32_t before = lanes_below(b);
    uint32_t total  = 0;
    for (int w = 0; w < RADIX / WAVE; ++w) {
      const uint32_t c = s_wcount[w];
      before += (w < wave) ? c : 0u;
      total += c;
    }
    // rank among the occurring values (<= 255); harmless in the (cleared) plan if it stays disabled
    plan->lut[p][tid] = static_cast<uint8_t>(before);
    if (tid == 0) {
      s_distinct[p] = total;
    }
    __syncthreads();
  }

  if (tid == 0) {
    // greedy grouping from the least significant position; positions with one value drop out
    uint32_t groups = 0, busy = 0, bits_in_group = 0;
    VirtGroup g{};
    for (uint32_t p = 0; p < passes; ++p) {
      const uint32_t d = s_distinct[p];
      if (d <= 1) {
        continue;
      }
      ++busy;
      const uint32_t bits = 32u - static_cast<uint32_t>(__builtin_clz(d - 1));  // ceil(log2 d), d >= 2
      if (g.count != 0 && bits_in_group + bits > RADIX_BITS) {
        plan->group[groups++] = g;
        g                     = VirtGroup{};
        bits_in_group         = 0;
      }
      g.pos[g.count]   = p;
      g.shift[g.count] = bits_in_group;
      ++g.count;
      bits_in_group += bits;
    }
    if (g.count != 0) {
      plan->group[groups++] = g;
    }
    // A pass on virtual digits costs about 1.12 ordinary passes (two table lookups per byte
    // position and key) and the second histogram sweep about 0.9: worth it when
    // 1.125 * groups + 0.875 < busy.
    const uint32_t enabled = (9u * groups + 7u < 8u * busy) ? 1u : 0u;
    plan->enabled          = enabled;
    plan->n_groups         = groups;
    s_enabled              = enabled;
    s_groups               = groups;
  }
  __syncthreads();
  if (s_enabled == 0) {
    return;
  }
  if (tid < static_cast<int>(passes)) {
    varying[tid] = 0;
  }
  for (uint32_t g = 0; g < s_groups; ++g) {
    hist[static_cast<uint64_t>(g) * RADIX + tid] = 0;
  }
}

// The virtual digit of one ordered key for one group.  `lut` (LDS): one table per position of
// the group, in group order, each code already shifted to its place inside the digit;
// `bit_offsets`: 8 bits per position, the bit offset of its byte in the ordered key (uniform,
// so that the loop control and the offsets stay on the scalar unit).
__device__ __forceinline__ uint32_t virtual_digit(uint64_t ordered, uint32_t count, uint64_t bit_offsets,
                                                   const uint8_t* lut)
{
  uint32_t d = 0;
  for (uint32_t j = 0; j < count; ++j) {
    const uint32_t off  = static_cast<uint32_t>(bit_offsets >> (8 * j)) & 0xFFu;
    const uint32_t byte = static_cast<uint32_t>(ordered >> off) & 0xFFu;
    d |= lut[j * RADIX + byte];
  }
  return d;
}

// Histograms of the virtual digits: hist[g][256] += counts over the row (cleared by
// vplan_kernel).  Exits at once when the plan is not enabled.
constexpr int VHIST_BLOCK = 256;
template <typename KeyT, int CODEC, typename OffT>
__global__ __launch_bounds__(VHIST_BLOCK) void vhist_kernel(const KeyT* __restrict__ keys,
                                                             OffT* __restrict__ hist,
                                                             const VirtPlan* __restrict__ plan,
                                                             uint64_t seg,
                                                             uint64_t chunk)
{
  constexpr int COPIES    = 4;
  constexpr int POSITIONS = static_cast<int>(sizeof(KeyT));  // byte positions of the ordered key
  static_assert(POSITIONS <= VIRT_MAX_POSITIONS, "keys of at most 8 bytes");
  __shared__ uint32_t s_hist[VIRT_MAX_POSITIONS * RADIX * COPIES];
  // per byte position: byte value -> code, already shifted to its place inside the digit of its
  // group (all zero for positions that belong to no group)
  __shared__ uint8_t s_tab[VIRT_MAX_POSITIONS * RADIX];
  __shared__ uint32_t s_ends;  // bit p: position p is the last one of its group
  if (plan->enabled == 0) {
    return;
  }
  const int tid         = threadIdx.x;
  const uint32_t groups = plan->n_groups;
  for (int j = tid; j < VIRT_MAX_POSITIONS * RADIX * COPIES; j += VHIST_BLOCK) {
    s_hist[j] = 0;
  }
  for (int j = tid; j < VIRT_MAX_POSITIONS * RADIX; j += VHIST_BLOCK) {
    s_tab[j] = 0;
  }
  __syncthreads();
  uint32_t ends = 0;
  for (uint32_t g = 0; g < groups; ++g) {
    const VirtGroup& grp = plan->group[g];
    for (uint32_t j = 0; j < grp.count; ++j) {
      const uint32_t p = grp.pos[j];
      s_tab[p * RADIX + tid] = static_cast<uint8_t>(plan->lut[p][tid] << grp.shift[j]);  // VHIST_BLOCK == RADIX
    }
    ends |= 1u << grp.pos[grp.count - 1];
  }
  static_assert(VHIST_BLOCK == RADIX, "one thread per table entry");
  if (tid == 0) {
    s_ends = ends;
  }
  __syncthreads();
  ends = s_ends;
  const uint64_t begin = static_cast<uint64_t>(blockIdx.x) * chunk;
  uint64_t end         = begin + chunk;
  if (end > seg) {
    end = seg;
  }
  // Few distinct digits is the very case this kernel runs in: the lanes of a wave spread their
  // LDS atomics over COPIES counters per digit value so that they do not pile up on a handful.
  const uint32_t copy = tid % COPIES;
  auto count_key = [&](KeyT raw) {
    uint64_t w[1];
    KeyTraits<CODEC, KeyT>::words(raw, w);
    uint32_t acc = 0, g = 0;
#pragma unroll
    for (int p = 0; p < POSITIONS; ++p) {
      acc |= s_tab[p * RADIX + (static_cast<uint32_t>(w[0] >> (p * RADIX_BITS)) & 0xFFu)];
      if ((ends >> p) & 1u) {  // uniform
        atomicAdd(&s_hist[(g * RADIX + acc) * COPIES + copy], 1u);
        acc = 0;
        ++g;
      }
    }
  };
  // four keys per thread and step, their loads issued together
  uint64_t i = begin + tid;
  for (; i + 3 * VHIST_BLOCK < end; i += 4 * VHIST_BLOCK) {
    const KeyT k0 = keys[i], k1 = keys[i + VHIST_BLOCK], k2 = keys[i + 2 * VHIST_BLOCK], k3 = keys[i + 3 * VHIST_BLOCK];
    count_key(k0);
    count_key(k1);
    count_key(k2);
    count_key(k3);
  }
  for (; i < end; i += VHIST_BLOCK) {
    count_key(keys[i]);
  }
  __syncthreads();
  for (uint32_t j = tid; j < groups * RADIX; j += VHIST_BLOCK) {
    uint32_t c = 0;
#pragma unroll
    for (int r = 0; r < COPIES; ++r) {
      c += s_hist[j * COPIES + r];
    }
    if (c != 0) {
      __hip_atomic_fetch_add(&hist[j], static_cast<OffT>(c), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
}

}  // namespace cpn
