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
//
// Distinct keys: when the whole row holds at most 256 different keys, ONE pass sorts it, on
// the rank of each key among the different keys.  Before the histogram sweep a sample of 4096
// keys is looked at (distinct_sample_kernel); unless it already holds more than 256 different
// keys, a sweep of its own collects the different keys and their counts in a hash table
// (distinct_sweep_kernel: per workgroup in LDS, merged into a table in the workspace; it stops
// at the 257th key) and distinct_plan_kernel ranks them, writes the offsets of the one pass
// and the lookup table in which the scatter pass finds every key's rank (copied into LDS).
// The histogram sweep and the other plan kernels then exit at once; when the table stays
// incomplete they run as if nothing had happened.
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

enum VirtMode : uint32_t { VIRT_OFF = 0, VIRT_GROUPS = 1, VIRT_DISTINCT = 2 };

struct VirtPlan {
  uint32_t enabled;   // VirtMode; VIRT_OFF: ordinary byte passes
  uint32_t n_groups;  // virtual passes, one per group, least significant first
  VirtGroup group[VIRT_MAX_POSITIONS];
  uint8_t lut[VIRT_MAX_POSITIONS][RADIX];  // per byte position: byte value -> code
};
constexpr uint64_t VIRT_PLAN_BYTES = 4096;
static_assert(sizeof(VirtPlan) <= VIRT_PLAN_BYTES, "plan does not fit its workspace slot");

// ---- distinct keys ----
// Keys are held as their ordered images; image 0 (the smallest possible key) marks an empty
// slot and is counted apart: when present its rank is 0.
constexpr uint32_t DISTINCT_MAX        = RADIX;  // more different keys than this: not used
constexpr uint32_t DISTINCT_SLOTS      = 1024;   // collecting table in the workspace
constexpr uint32_t DISTINCT_LOCAL      = 512;    // collecting table of a workgroup (LDS)
constexpr uint32_t DISTINCT_COPIES     = 4;      // counters per slot of the LDS table, selected by lane
constexpr uint32_t DISTINCT_LOOKUP     = 512;    // table of the scatter pass, at most half full
constexpr uint32_t DISTINCT_MAX_PROBES = 64;     // longer chains: give up (every loop below is bounded)

struct DistinctTable {
  uint64_t keys[DISTINCT_SLOTS];    // 0: empty
  uint32_t counts[DISTINCT_SLOTS];  // occurrences in the row
  uint64_t lookup_keys[DISTINCT_LOOKUP];
  uint8_t lookup_rank[DISTINCT_LOOKUP];
  uint32_t n_keys;      // slots taken
  uint32_t overflow;    // more than DISTINCT_MAX keys, or a chain too long: the table is incomplete
  uint32_t zero_count;  // occurrences of image 0
  uint32_t sample_many; // a sample of the row already holds too many keys: nothing is collected
};
constexpr uint64_t DISTINCT_TABLE_BYTES = 20480;
static_assert(sizeof(DistinctTable) <= DISTINCT_TABLE_BYTES, "table does not fit its workspace slot");
constexpr uint64_t VIRT_WORKSPACE_BYTES = VIRT_PLAN_BYTES + DISTINCT_TABLE_BYTES;

__device__ __forceinline__ uint32_t distinct_hash(uint64_t image, uint32_t slots_log2)
{
  const uint32_t x = static_cast<uint32_t>(image) ^ static_cast<uint32_t>(image >> 32) * 0x85EBCA6Bu;
  return (x * 0x9E3779B1u) >> (32u - slots_log2);
}

// Rank of a key of the row, from the lookup table in LDS (every key of the row is in it).
__device__ __forceinline__ uint32_t distinct_rank(uint64_t image, const uint64_t* lookup_keys,
                                                   const uint8_t* lookup_rank)
{
  if (image == 0) {
    return 0;
  }
  uint32_t h = distinct_hash(image, 9);
  static_assert(DISTINCT_LOOKUP == 512, "hash width");
  for (uint32_t probe = 0; probe < DISTINCT_MAX_PROBES && lookup_keys[h] != image; ++probe) {
    h = (h + 1) & (DISTINCT_LOOKUP - 1);
  }
  return lookup_rank[h];
}

// The workgroup stops collecting; the first thread to say so also raises `told`, a word of the row's table (one
// store per workgroup: stores of many threads to that one word would queue up in L2).
__device__ __forceinline__ void distinct_give_up(uint32_t* state, uint32_t* told)
{
  if (atomicExch(&state[1], 1u) == 0) {
    __hip_atomic_store(told, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}

// Collects the different keys of a workgroup's share of the row: LDS table `keys` of
// DISTINCT_LOCAL slots with DISTINCT_COPIES counters each in `counts` (cleared by the caller;
// the few keys of such a row would otherwise queue on one counter each), `state[0]` = slots
// taken, `state[1]` = gave up, `state[2]` = occurrences of image 0.
// Giving up is also told to the row's table at once (`told`), so that workgroups starting later
// do not try.
__device__ __forceinline__ void distinct_collect(uint64_t image, uint64_t* keys, uint32_t* counts, uint32_t* state,
                                                  uint32_t copy, uint32_t* told)
{
  if (image == 0) {
    atomicAdd(&state[2], 1u);
    return;
  }
  uint32_t h = distinct_hash(image, 9);
  static_assert(DISTINCT_LOCAL == 512, "hash width");
  for (uint32_t probe = 0; probe < DISTINCT_MAX_PROBES; ++probe) {
    uint64_t cur = __hip_atomic_load(&keys[h], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    if (cur == 0) {
      cur = atomicCAS(reinterpret_cast<unsigned long long*>(&keys[h]), 0ull, static_cast<unsigned long long>(image));
      if (cur == 0) {
        // a few more keys per thread go in after the limit is passed (the caller re-reads
        // state[1] every few keys); should the table fill up, the bound on the probes ends
        // the search
        if (atomicAdd(&state[0], 1u) >= DISTINCT_MAX) {
          distinct_give_up(state, told);
        }
        cur = image;
      }
    }
    if (cur == image) {
      atomicAdd(&counts[h * DISTINCT_COPIES + copy], 1u);
      return;
    }
    h = (h + 1) & (DISTINCT_LOCAL - 1);
  }
  distinct_give_up(state, told);
}

// One collected key (with its count) into the table of the workspace.
__device__ __forceinline__ void distinct_merge(uint64_t image, uint32_t count, DistinctTable* table)
{
  uint32_t h = distinct_hash(image, 10);
  static_assert(DISTINCT_SLOTS == 1024, "hash width");
  for (uint32_t probe = 0; probe < DISTINCT_MAX_PROBES; ++probe) {
    if (__hip_atomic_load(&table->overflow, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0) {
      return;
    }
    unsigned long long* slot = reinterpret_cast<unsigned long long*>(&table->keys[h]);
    uint64_t cur             = __hip_atomic_load(slot, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (cur == 0) {
      cur = atomicCAS(slot, 0ull, static_cast<unsigned long long>(image));
      if (cur == 0) {
        if (atomicAdd(&table->n_keys, 1u) >= DISTINCT_MAX) {
          __hip_atomic_store(&table->overflow, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        cur = image;
      }
    }
    if (cur == image) {
      atomicAdd(&table->counts[h], count);
      return;
    }
    h = (h + 1) & (DISTINCT_SLOTS - 1);
  }
  if (__hip_atomic_load(&table->overflow, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == 0) {
    __hip_atomic_store(&table->overflow, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}

// One workgroup: DISTINCT_SAMPLE keys from all over the row; more than DISTINCT_MAX different
// ones among them raise table->sample_many.
constexpr uint32_t DISTINCT_SAMPLE = 4096;
template <typename KeyT, int CODEC>
__global__ __launch_bounds__(RADIX) void distinct_sample_kernel(const KeyT* __restrict__ keys,
                                                                 uint64_t seg,
                                                                 DistinctTable* __restrict__ table)
{
  __shared__ uint64_t s_keys[DISTINCT_LOCAL];
  __shared__ uint32_t s_counts[DISTINCT_LOCAL * DISTINCT_COPIES];
  __shared__ uint32_t s_state[3];
  const uint32_t tid = threadIdx.x;
  for (uint32_t j = tid; j < DISTINCT_LOCAL; j += RADIX) {
    s_keys[j] = 0;
  }
  for (uint32_t j = tid; j < DISTINCT_LOCAL * DISTINCT_COPIES; j += RADIX) {
    s_counts[j] = 0;
  }
  if (tid < 3) {
    s_state[tid] = 0;
  }
  __syncthreads();
  // DISTINCT_SAMPLE / WAVE runs of WAVE neighbouring keys, the runs spread evenly over the row (few
  // memory pages are touched, every wave reads one run per step)
  const uint64_t n      = seg < DISTINCT_SAMPLE ? seg : DISTINCT_SAMPLE;
  const uint64_t stride = (seg / n) * WAVE;  // from run to run
  constexpr int PER_THREAD = DISTINCT_SAMPLE / RADIX;
  KeyT mine[PER_THREAD];  // all loads of a thread are issued before the first key is looked at
#pragma unroll
  for (int j = 0; j < PER_THREAD; ++j) {
    const uint64_t i = static_cast<uint64_t>(j) * RADIX + tid;
    mine[j]          = (i < n) ? keys[(i / WAVE) * stride + (i % WAVE)] : KeyT{};
  }
#pragma unroll
  for (int j = 0; j < PER_THREAD; ++j) {
    const uint64_t i = static_cast<uint64_t>(j) * RADIX + tid;
    if (i < n && *static_cast<volatile uint32_t*>(&s_state[1]) == 0) {
      uint64_t w[KeyTraits<CODEC, KeyT>::NWORDS];
      KeyTraits<CODEC, KeyT>::words(mine[j], w);
      distinct_collect(w[0], s_keys, s_counts, s_state, tid % DISTINCT_COPIES, &table->sample_many);
    }
  }
}

// The collecting sweep: every workgroup gathers the different keys of its chunk of the row (and how
// often each occurs) in LDS and merges them into the row's table.  Exits at once when the sample
// already found too many; workgroups that start after one has given up do not try either.
constexpr int DSWEEP_BLOCK = 256;
template <typename KeyT, int CODEC>
__global__ __launch_bounds__(DSWEEP_BLOCK) void distinct_sweep_kernel(const KeyT* __restrict__ keys,
                                                                       uint64_t seg,
                                                                       uint64_t chunk,
                                                                       DistinctTable* __restrict__ table)
{
  static_assert(KeyTraits<CODEC, KeyT>::NWORDS == 1, "distinct keys: one ordered word");
  if (table->sample_many != 0) {
    return;
  }
  __shared__ uint64_t s_keys[DISTINCT_LOCAL];
  __shared__ uint32_t s_counts[DISTINCT_LOCAL * DISTINCT_COPIES];
  __shared__ uint32_t s_state[3];  // slots taken, gave up, occurrences of image 0
  const uint32_t tid = threadIdx.x;
  for (uint32_t j = tid; j < DISTINCT_LOCAL; j += DSWEEP_BLOCK) {
    s_keys[j] = 0;
  }
  for (uint32_t j = tid; j < DISTINCT_LOCAL * DISTINCT_COPIES; j += DSWEEP_BLOCK) {
    s_counts[j] = 0;
  }
  if (tid == 0) {
    s_state[0] = 0;
    s_state[1] = __hip_atomic_load(&table->overflow, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    s_state[2] = 0;
  }
  __syncthreads();
  const uint64_t begin = static_cast<uint64_t>(blockIdx.x) * chunk;
  uint64_t end         = begin + chunk;
  if (end > seg) {
    end = seg;
  }
  const uint32_t copy = tid % DISTINCT_COPIES;
  auto collect = [&](KeyT raw) {
    uint64_t w[1];
    KeyTraits<CODEC, KeyT>::words(raw, w);
    distinct_collect(w[0], s_keys, s_counts, s_state, copy, &table->overflow);
  };
  // four keys per thread and step, their loads issued together; has the workgroup given up is
  // asked once per step
  uint64_t i = begin + tid;
  for (; i + 3 * DSWEEP_BLOCK < end; i += 4 * DSWEEP_BLOCK) {
    if (*static_cast<volatile uint32_t*>(&s_state[1]) != 0) {
      break;
    }
    const KeyT k0 = keys[i], k1 = keys[i + DSWEEP_BLOCK], k2 = keys[i + 2 * DSWEEP_BLOCK], k3 = keys[i + 3 * DSWEEP_BLOCK];
    collect(k0);
    collect(k1);
    collect(k2);
    collect(k3);
  }
  for (; i < end; i += DSWEEP_BLOCK) {
    if (*static_cast<volatile uint32_t*>(&s_state[1]) != 0) {
      break;
    }
    collect(keys[i]);
  }
  __syncthreads();
  if (s_state[1] != 0) {
    return;  // whoever gave up has said so in the table
  }
  for (uint32_t j = tid; j < DISTINCT_LOCAL; j += DSWEEP_BLOCK) {
    if (s_keys[j] != 0) {
      uint32_t c = 0;
#pragma unroll
      for (uint32_t r = 0; r < DISTINCT_COPIES; ++r) {
        c += s_counts[j * DISTINCT_COPIES + r];
      }
      distinct_merge(s_keys[j], c, table);
    }
  }
  if (tid == 0 && s_state[2] != 0) {
    atomicAdd(&table->zero_count, s_state[2]);
  }
}

// One workgroup of 256 threads, after the collecting sweep.  When the table is complete (at most
// 256 different keys): ranks them, writes the offsets of the one pass into hist[0][*], the lookup
// table of the scatter pass, varying[] (pass 0 runs unless all keys are equal) and
// plan->enabled = VIRT_DISTINCT, after which the histogram sweep and the other plan kernels have
// nothing to do.  Otherwise (also when the counts do not add up to `seg`) leaves everything alone.
template <typename OffT>
__global__ __launch_bounds__(RADIX) void distinct_plan_kernel(OffT* __restrict__ hist,
                                                               uint32_t* __restrict__ varying,
                                                               VirtPlan* __restrict__ plan,
                                                               DistinctTable* __restrict__ table,
                                                               uint64_t seg,
                                                               uint32_t passes)
{
  __shared__ uint64_t s_keys[DISTINCT_MAX];  // the row's different keys (other than image 0), unordered
  __shared__ uint32_t s_slot[DISTINCT_MAX];  // where each sits in the collecting table
  __shared__ uint32_t s_nkeys;
  __shared__ uint64_t s_lookup_keys[DISTINCT_LOOKUP];
  __shared__ uint8_t s_lookup_rank[DISTINCT_LOOKUP];
  __shared__ OffT s_count[RADIX];
  __shared__ OffT s_wsum[RADIX / WAVE];
  __shared__ uint32_t s_use_table, s_failed, s_total;
  const int tid  = threadIdx.x;
  const int lane = tid & (WAVE - 1);
  const int wave = tid / WAVE;
  if (tid == 0) {
    const uint32_t k = table->n_keys + (table->zero_count != 0 ? 1u : 0u);
    s_use_table      = (table->sample_many == 0 && table->overflow == 0 && k >= 1 && k <= DISTINCT_MAX) ? 1u : 0u;
    s_total          = k;
    s_failed         = 0;
    s_nkeys          = 0;
  }
  __syncthreads();
  if (s_use_table == 0) {
    return;
  }
  const uint32_t zero_rank = (table->zero_count != 0) ? 1u : 0u;
  for (uint32_t j = tid; j < DISTINCT_SLOTS; j += RADIX) {
    const uint64_t key = table->keys[j];
    if (key != 0) {
      const uint32_t i = atomicAdd(&s_nkeys, 1u);
      if (i < DISTINCT_MAX) {  // n_keys <= DISTINCT_MAX was checked above
        s_keys[i] = key;
        s_slot[i] = j;
      }
    }
  }
  for (uint32_t j = tid; j < DISTINCT_LOOKUP; j += RADIX) {
    s_lookup_keys[j] = 0;
    s_lookup_rank[j] = 0;
  }
  s_count[tid] = (tid == 0) ? static_cast<OffT>(table->zero_count) : static_cast<OffT>(0);
  __syncthreads();
  const uint32_t nkeys = (s_nkeys < DISTINCT_MAX) ? s_nkeys : DISTINCT_MAX;
  if (static_cast<uint32_t>(tid) < nkeys) {  // RADIX threads, DISTINCT_MAX == RADIX keys at most
    const uint64_t key = s_keys[tid];
    uint32_t rank      = zero_rank;
    for (uint32_t i = 0; i < nkeys; ++i) {
      rank += (s_keys[i] < key) ? 1u : 0u;
    }
    s_count[rank] = static_cast<OffT>(table->counts[s_slot[tid]]);  // ranks are distinct: one writer each
    uint32_t h    = distinct_hash(key, 9);
    bool placed   = false;
    for (uint32_t probe = 0; probe < DISTINCT_MAX_PROBES && !placed; ++probe) {
      const uint64_t prev =
        atomicCAS(reinterpret_cast<unsigned long long*>(&s_lookup_keys[h]), 0ull, static_cast<unsigned long long>(key));
      if (prev == 0) {
        s_lookup_rank[h] = static_cast<uint8_t>(rank);
        placed           = true;
      } else {
        h = (h + 1) & (DISTINCT_LOOKUP - 1);
      }
    }
    if (!placed) {
      s_failed = 1;  // a chain the scatter pass would not follow to its end
    }
  }
  __syncthreads();
  if (s_failed != 0) {
    return;  // the byte passes take over
  }
  {
    // exclusive scan of the counts by rank: the offsets of the one pass
    const OffT c = s_count[tid];
    OffT incl    = c;
#pragma unroll
    for (int delta = 1; delta < WAVE; delta <<= 1) {
      const OffT t = __shfl_up(incl, delta, WAVE);
      if (lane >= delta) {
        incl += t;
      }
    }
    if (lane == WAVE - 1) {
      s_wsum[wave] = incl;
    }
    __syncthreads();
    OffT prefix = 0;
    for (int w = 0; w < wave; ++w) {
      prefix += s_wsum[w];
    }
    // the counts must add up to the row: offsets from a table that lost or doubled a key would
    // send the scatter pass out of the row, so such a table is not used
    if (tid == RADIX - 1 && static_cast<uint64_t>(prefix + incl) != seg) {
      s_failed = 1;
    }
    __syncthreads();
    if (s_failed != 0) {
      return;
    }
    hist[tid] = prefix + incl - c;
    for (uint32_t j = tid; j < DISTINCT_LOOKUP; j += RADIX) {
      table->lookup_keys[j] = s_lookup_keys[j];
      table->lookup_rank[j] = s_lookup_rank[j];
    }
    if (tid < static_cast<int>(passes)) {
      varying[tid] = (tid == 0 && s_total >= 2) ? 1u : 0u;  // one key only: nothing to sort
    }
    if (tid == 0) {
      plan->enabled  = VIRT_DISTINCT;
      plan->n_groups = 1;
    }
  }
}

// One workgroup of 256 threads.  `hist` holds the exclusive-scanned byte histograms of the one
// row ([pass][256]); `varying[p]` says whether position p differs between keys at all.
// When virtual digits save enough passes to pay for themselves: writes the plan, clears hist[g][*] for the
// groups (vhist_kernel accumulates there) and resets varying (the second scan raises it again
// for the groups).  Otherwise leaves everything alone with enabled == 0.  Nothing to do when the
// sort already runs on the ranks of the row's different keys.
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
  if (plan->enabled == VIRT_DISTINCT) {
    return;  // distinct_plan_kernel has settled everything; the byte histograms were not even made
  }
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
    const uint32_t enabled = (9u * groups + 7u < 8u * busy) ? VIRT_GROUPS : VIRT_OFF;
    plan->enabled          = enabled;
    plan->n_groups         = groups;
    s_enabled              = enabled;
    s_groups               = groups;
  }
  __syncthreads();
  if (s_enabled == VIRT_OFF) {
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
//
// count == VIRT_COUNT_DISTINCT: the pass runs on the ranks of the row's different keys; `lut`
// then holds the lookup table (DISTINCT_LOOKUP keys, then as many ranks).
constexpr uint32_t VIRT_COUNT_DISTINCT = 0xFFFFFFFFu;
constexpr uint32_t VIRT_LDS_BYTES      = DISTINCT_LOOKUP * 9;  // >= the tables of one group of virtual digits
static_assert(VIRT_LDS_BYTES >= VIRT_MAX_POSITIONS * RADIX, "LDS area of the scatter pass");
__device__ __forceinline__ uint32_t virtual_digit(uint64_t ordered, uint32_t count, uint64_t bit_offsets,
                                                   const uint8_t* lut)
{
  if (count == VIRT_COUNT_DISTINCT) {  // uniform
    return distinct_rank(ordered, reinterpret_cast<const uint64_t*>(lut), lut + DISTINCT_LOOKUP * 8);
  }
  uint32_t d = 0;
  for (uint32_t j = 0; j < count; ++j) {
    const uint32_t off  = static_cast<uint32_t>(bit_offsets >> (8 * j)) & 0xFFu;
    const uint32_t byte = static_cast<uint32_t>(ordered >> off) & 0xFFu;
    d |= lut[j * RADIX + byte];
  }
  return d;
}

// Histograms of the virtual digits: hist[g][256] += counts over the row (cleared by
// vplan_kernel).  Exits at once unless the plan runs on grouped virtual digits.
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
  if (plan->enabled != VIRT_GROUPS) {
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
