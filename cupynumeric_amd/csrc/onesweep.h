// Global LSD radix sort ("onesweep"): one histogram sweep over the keys, then one
// scatter kernel per 8-bit digit in which every workgroup sorts a tile through LDS and
// finds its global offsets with a decoupled look-back over per-tile descriptors.
//
// Replaces cub::DeviceRadixSort::SortKeys / SortPairs and, for rows too long for LDS,
// cub::DeviceSegmentedRadixSort (src/cupynumeric/sort/cub_sort.cuh:60-182).  Rows are
// batched into the same launches: a tile never straddles two rows and the look-back
// stops at the first tile of its row.
//
// Data layout in HBM
//   keys      raw element bits, dense row-major, ping-ponged between caller/workspace buffers
//   payload   position of the element inside its row, 32-bit while a row is shorter than
//             2^30 elements (64-bit otherwise), synthesised by the first pass and widened
//             to int64 (+ index_offset) by the last one
//   hist      [row][pass][256] counts, exclusive-scanned in place
//   desc      [pass][tile][256] words: 2 status bits | count   (aggregate or inclusive)
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "radix_common.h"
#include "virtual_digits.h"

namespace cpn {

// Widths that depend on the row length.  Rows shorter than 2^30 keep every per-row count
// and the index payload in 32 bits (two bits of a descriptor word hold its status).
template <bool BIG>
struct RowWidth;
template <>
struct RowWidth<false> {
  using off_t = uint32_t;
};
template <>
struct RowWidth<true> {
  using off_t = uint64_t;
};

template <typename D>
struct DescBits {
  static constexpr int BITS    = sizeof(D) * 8;
  static constexpr D AGGREGATE = static_cast<D>(1) << (BITS - 2);
  static constexpr D INCLUSIVE = static_cast<D>(2) << (BITS - 2);
  static constexpr D STATUS    = static_cast<D>(3) << (BITS - 2);
  static constexpr D VALUE     = static_cast<D>(~STATUS);
};

// Upper bound on polls of one descriptor before a tile gives up and flags an error, so
// that every wave exits even if a predecessor never publishes.
constexpr uint32_t LOOKBACK_SPIN_LIMIT = 1u << 22;
// The limit in force: LOOKBACK_SPIN_LIMIT unless changed by cpn_set_lookback_spin_limit (tests of
// the failure path set it to 1, so that a tile gives up at its first unanswered poll).
uint32_t lookback_spin_limit();

// Predecessor descriptors each look-back round reads at once.
#ifndef CPN_LOOKBACK_WINDOW
#define CPN_LOOKBACK_WINDOW 4
#endif
constexpr int LOOKBACK_WINDOW = CPN_LOOKBACK_WINDOW;

// Status word values written by kernels into the workspace header.
constexpr uint32_t DEVICE_ERR_LOOKBACK = 1u;

// ---------------------------------------------------------------------------------------
// zero fill (capture-safe replacement for a memset node)
// ---------------------------------------------------------------------------------------
static __global__ __launch_bounds__(256) void zero_fill_kernel(uint4* p, uint64_t n_vec)
{
  const uint64_t stride = static_cast<uint64_t>(gridDim.x) * blockDim.x;
  for (uint64_t i = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n_vec; i += stride) {
    p[i] = make_uint4(0u, 0u, 0u, 0u);
  }
}

// ---------------------------------------------------------------------------------------
// histogram sweep: all digit histograms of every row in one read of the keys
// ---------------------------------------------------------------------------------------
constexpr int HIST_BLOCK = 256;
// Copies of every counter, selected by lane: keys of one wave that share a digit (the top
// digit of floats takes a handful of values) then spread over several LDS banks instead of
// queueing on one address.
// Measured on 2^28 float32 keys: 1 copy 0.51 ms, 2: 0.37, 4: 0.30, 8: 0.27 ms (4.0 TB/s; a plain
// read-only sweep of the same buffer takes 0.15 ms, so the four LDS atomics per key remain the
// bound).  64-bit keys have twice the histograms: 4 copies keep the block at 32 KiB of LDS
// (complex keys: 9 passes x 4 copies, 17 passes x 2 copies).
__host__ __device__ constexpr int hist_copies(int passes) { return passes <= 4 ? 8 : (passes <= 9 ? 4 : 2); }

// Returns whether `raw` is a float key whose bits are not determined by its place in the order
// (a NaN or a -0.0); false for every other key type.
template <typename KeyT, int CODEC, int PASSES, bool SPECIALS>
__device__ __forceinline__ bool hist_accumulate(uint32_t* s_hist, KeyT raw, uint32_t copy)
{
  using KT                  = KeyTraits<CODEC, KeyT>;
  constexpr int HIST_COPIES = hist_copies(PASSES);
  uint64_t w[KT::NWORDS];
  KT::words(raw, w);
  bool special = false;
  if constexpr (SPECIALS) {
    special = static_cast<KeyT>(w[0]) != sign_flip(raw);
  }
#pragma unroll
  for (int p = 0; p < PASSES; ++p) {
    const uint32_t d = static_cast<uint32_t>(w[p / 8] >> ((p % 8) * RADIX_BITS)) & 0xFFu;
    atomicAdd(&s_hist[(p * RADIX + d) * HIST_COPIES + copy], 1u);
  }
  return special;
}

// grid = rows * blocks_per_row; block b of a row covers elements [b*chunk, min(seg, (b+1)*chunk)).
// 128-bit loads over the 16-byte aligned middle of the chunk, scalar head and tail.
// `vplan` (may be null): nothing to do when the sort already runs on the ranks of the row's
// different keys (virtual_digits.h).
// SPECIALS (float keys, keys-only sorts): also tells through `specials` whether a NaN or a -0.0 occurs.
template <typename KeyT, int CODEC, typename OffT, bool SPECIALS = false>
__global__ __launch_bounds__(HIST_BLOCK) void histogram_kernel(const KeyT* __restrict__ keys,
                                                                 OffT* __restrict__ hist,
                                                                 uint64_t seg,
                                                                 uint32_t blocks_per_row,
                                                                 uint64_t chunk,
                                                                 const VirtPlan* __restrict__ vplan,
                                                                 uint32_t* __restrict__ specials)
{
  constexpr int PASSES      = KeyTraits<CODEC, KeyT>::PASSES;
  constexpr int VEC         = 16 / sizeof(KeyT);
  constexpr int HIST_COPIES = hist_copies(PASSES);
  if (vplan != nullptr && vplan->enabled == VIRT_DISTINCT) {
    return;
  }
  __shared__ uint32_t s_hist[PASSES * RADIX * HIST_COPIES];

  const int tid        = threadIdx.x;
  const uint32_t copy  = tid % HIST_COPIES;
  const uint64_t row   = blockIdx.x / blocks_per_row;
  const uint32_t piece = blockIdx.x - static_cast<uint32_t>(row * blocks_per_row);
  const uint64_t begin = static_cast<uint64_t>(piece) * chunk;
  uint64_t end         = begin + chunk;
  if (end > seg) {
    end = seg;
  }
  for (int j = tid; j < PASSES * RADIX * HIST_COPIES; j += HIST_BLOCK) {
    s_hist[j] = 0;
  }
  __syncthreads();
  bool special = false;  // float keys: a NaN or a -0.0 among this thread's keys

  if (begin < end) {
    const KeyT* p = keys + row * seg;
    // elements before the first 16-byte boundary
    const uintptr_t addr = reinterpret_cast<uintptr_t>(p + begin);
    uint64_t head        = ((16u - (addr & 15u)) & 15u) / sizeof(KeyT);
    if (head > end - begin) {
      head = end - begin;
    }
    for (uint64_t i = tid; i < head; i += HIST_BLOCK) {
      special |= hist_accumulate<KeyT, CODEC, PASSES, SPECIALS>(s_hist, p[begin + i], copy);
    }
    const uint64_t vbegin = begin + head;
    const uint64_t nvec   = (end - vbegin) / VEC;
    const uint4* vp       = reinterpret_cast<const uint4*>(p + vbegin);
    uint64_t v            = tid;
    // two 128-bit loads in flight per thread
    for (; v + HIST_BLOCK < nvec; v += 2 * HIST_BLOCK) {
      const uint4 q0 = vp[v];
      const uint4 q1 = vp[v + HIST_BLOCK];
      KeyT k[2 * VEC];
      __builtin_memcpy(k, &q0, 16);
      __builtin_memcpy(k + VEC, &q1, 16);
#pragma unroll
      for (int j = 0; j < 2 * VEC; ++j) {
        special |= hist_accumulate<KeyT, CODEC, PASSES, SPECIALS>(s_hist, k[j], copy);
      }
    }
    for (; v < nvec; v += HIST_BLOCK) {
      const uint4 q = vp[v];
      KeyT k[VEC];
      __builtin_memcpy(k, &q, 16);
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        special |= hist_accumulate<KeyT, CODEC, PASSES, SPECIALS>(s_hist, k[j], copy);
      }
    }
    for (uint64_t i = vbegin + nvec * VEC + tid; i < end; i += HIST_BLOCK) {
      special |= hist_accumulate<KeyT, CODEC, PASSES, SPECIALS>(s_hist, p[i], copy);
    }
  }
  // (the barrier also ends the accumulation) `specials`: does any float key of the sort tie with
  // keys of other bits?  The first pass of a keys-only sort may ignore stability if not.
  if constexpr (SPECIALS) {
    const int any_special = __syncthreads_or(special ? 1 : 0);
    if (any_special != 0 && tid == 0) {
      __hip_atomic_store(specials, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  } else {
    __syncthreads();
  }

  OffT* out = hist + row * (PASSES * RADIX);
  for (int j = tid; j < PASSES * RADIX; j += HIST_BLOCK) {
    uint32_t c = 0;
#pragma unroll
    for (int r = 0; r < HIST_COPIES; ++r) {
      c += s_hist[j * HIST_COPIES + r];
    }
    if (c != 0) {
      __hip_atomic_fetch_add(&out[j], static_cast<OffT>(c), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
}

// ---------------------------------------------------------------------------------------
// pass plan: which passes run and between which buffers, decided on the device
// ---------------------------------------------------------------------------------------
// Passes whose digit is the same for all keys of every row are skipped.  Which buffer a pass
// reads and writes then depends on how many passes remain, which only the device knows after
// the histogram sweep: a one-thread kernel writes one PassPlan per pass and the scatter
// kernels look their buffers up by id.  The last running pass always writes the caller's
// arrays; the ones before it alternate, walking backwards, between two scratch buffers.
constexpr int MAX_PASSES = 24;
enum KeyBuf : uint32_t { KEY_IN = 0, KEY_OUT = 1, KEY_T1 = 2, KEY_T2 = 3 };
enum IdxBuf : uint32_t { IDX_FINAL = 1, IDX_T1 = 2, IDX_ALIAS = 3 };  // ALIAS: the int64 output used as narrow scratch
constexpr uint32_t BUF_NONE = 0xFFu;

struct PassPlan {
  uint32_t active;   // 0: the pass exits at once
  uint32_t key_src;  // KeyBuf
  uint32_t key_dst;  // KeyBuf or BUF_NONE (index-only sort, last pass)
  uint32_t idx_src;  // IdxBuf or BUF_NONE (first running pass: positions are synthesised)
  uint32_t idx_dst;  // IdxBuf
  uint32_t first;    // bit 0: first running pass; bit 1: that pass need not be stable (PLAN_FREE_RANK)
};
constexpr uint32_t PLAN_FIRST     = 1u;
constexpr uint32_t PLAN_FREE_RANK = 2u;

struct SortPlan {
  PassPlan pass[MAX_PASSES];
  uint32_t n_active;
  // Keys-only sorts of float keys without a NaN or a -0.0 (the histogram sweep has looked): the order-
  // preserving image is then a bijection of the bits, so the first running pass stores the images,
  // every pass takes plain bytes of them as digits, and the last pass maps them back as it stores
  // (saves the key transform twice per key and pass; see onesweep_tile, UNFLIP).
  uint32_t flipped;
};

struct PlanRequest {
  uint32_t passes;
  uint32_t want_values;
  uint32_t want_indices;
  uint32_t in_place;
  // Keys-only sorts: the first running pass need not be stable when keys that tie in every digit
  // are the same bits: always for integer keys (free_rank = 1, specials = nullptr); for float
  // keys unless the histogram sweep met a NaN or a -0.0 (*specials != 0).
  uint32_t free_rank;
  const uint32_t* specials;
};

// One thread.  `varying` is read with device-scope loads: the flags may have been raised by other
// workgroups of the same launch (make_plan at the end of the scan kernel).
__device__ __forceinline__ void make_plan(const uint32_t* varying, SortPlan* __restrict__ plan, PlanRequest rq)
{
  uint32_t flags = 0;  // bit p: pass p runs
  uint32_t k     = 0;
  for (uint32_t p = 0; p < rq.passes; ++p) {
    if (__hip_atomic_load(&varying[p], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0) {
      flags |= 1u << p;
      ++k;
    }
  }
  plan->n_active = k;
  plan->flipped  = (rq.free_rank != 0 && rq.specials != nullptr && rq.want_indices == 0 &&
                   __hip_atomic_load(rq.specials, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == 0)
                     ? 1u
                     : 0u;
  // scratch partner of T1: the caller's value array when it is free to be overwritten early
  const uint32_t key_x = (rq.want_values && !rq.in_place) ? KEY_OUT : KEY_T2;
  uint32_t j = 0, key_prev = KEY_IN, idx_prev = BUF_NONE;
  for (uint32_t p = 0; p < rq.passes; ++p) {
    PassPlan e{};
    if ((flags >> p) & 1u) {
      ++j;
      const uint32_t from_last = k - j;
      e.active                 = 1;
      e.first                  = (j == 1) ? PLAN_FIRST : 0u;
      if (j == 1 && rq.free_rank != 0 &&
          (rq.specials == nullptr || __hip_atomic_load(rq.specials, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == 0)) {
        e.first |= PLAN_FREE_RANK;
      }
      e.key_src                = key_prev;
      e.idx_src                = idx_prev;
      if (from_last == 0) {
        e.key_dst = rq.want_values ? ((k == 1 && rq.in_place) ? KEY_T1 : KEY_OUT) : BUF_NONE;
        e.idx_dst = IDX_FINAL;
      } else {
        e.key_dst = (from_last & 1u) ? KEY_T1 : key_x;
        e.idx_dst = (from_last & 1u) ? IDX_T1 : IDX_ALIAS;
      }
      key_prev = e.key_dst;
      idx_prev = e.idx_dst;
    }
    plan->pass[p] = e;
  }
}

static __global__ void plan_kernel(const uint32_t* __restrict__ varying, SortPlan* __restrict__ plan, PlanRequest rq)
{
  if (threadIdx.x == 0 && blockIdx.x == 0) {
    make_plan(varying, plan, rq);
  }
}

// Exclusive scan of every 256-bin histogram in place, one wavefront per (row, pass) histogram
// (four bins per lane), the wavefronts of the grid striding over the histograms: a request of
// many short rows has as many histograms as rows x passes, and one workgroup each, with one
// device-scope atomic each for the plan, took longer than the scatter passes.  A pass on whose
// digit all keys of a row agree (one bin holds the whole row) would be the identity permutation
// for that row; `varying[pass]` is raised by every row for which that is not so.
constexpr int SCAN_BLOCK = 256;
template <typename OffT>
__global__ __launch_bounds__(SCAN_BLOCK) void histogram_scan_kernel(OffT* __restrict__ hist,
                                                                    uint32_t* __restrict__ varying,
                                                                    uint64_t seg,
                                                                    uint32_t passes,
                                                                    uint64_t n_hist,
                                                                    const VirtPlan* __restrict__ vplan,
                                                                    uint32_t second,
                                                                    uint32_t* __restrict__ blocks_done,
                                                                    SortPlan* __restrict__ plan,
                                                                    PlanRequest rq)
{
  // first use (`second` == 0): nothing when the sort already runs on the ranks of the row's
  // different keys.  Second use, after vplan_kernel: scans the histograms of the grouped virtual
  // digits (one row, histogram = group) and nothing when that plan is not in force.
  if (vplan != nullptr) {
    const uint32_t mode = vplan->enabled;
    if (second == 0 ? (mode == VIRT_DISTINCT) : (mode != VIRT_GROUPS)) {
      return;
    }
    if (second != 0 && n_hist > vplan->n_groups) {
      n_hist = vplan->n_groups;
    }
  }
  constexpr int PER_LANE = RADIX / WAVE;
  const int tid          = threadIdx.x;
  const int lane         = tid & (WAVE - 1);
  const uint64_t wave    = static_cast<uint64_t>(blockIdx.x) * (SCAN_BLOCK / WAVE) + tid / WAVE;
  const uint64_t nwaves  = static_cast<uint64_t>(gridDim.x) * (SCAN_BLOCK / WAVE);
  uint32_t raised        = 0;  // passes this wavefront has flagged already
  for (uint64_t h = wave; h < n_hist; h += nwaves) {
    OffT* p = hist + h * RADIX + lane * PER_LANE;
    OffT c[PER_LANE];
    OffT sum     = 0;
    bool one_bin = false;
#pragma unroll
    for (int j = 0; j < PER_LANE; ++j) {
      c[j] = p[j];
      one_bin |= (c[j] == static_cast<OffT>(seg));
      sum += c[j];
    }
    const uint32_t pass = static_cast<uint32_t>(h % passes);
    if (__builtin_amdgcn_ballot_w64(one_bin) == 0 && ((raised >> pass) & 1u) == 0) {
      raised |= 1u << pass;
      if (lane == 0) {
        __hip_atomic_fetch_or(&varying[pass], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
    OffT incl = sum;
#pragma unroll
    for (int delta = 1; delta < WAVE; delta <<= 1) {
      const OffT t = __shfl_up(incl, delta, WAVE);
      if (lane >= delta) {
        incl += t;
      }
    }
    OffT run = incl - sum;
#pragma unroll
    for (int j = 0; j < PER_LANE; ++j) {
      p[j] = run;
      run += c[j];
    }
  }
  // `blocks_done` given: the block that finishes last also makes the pass plan (saves a launch)
  if (blocks_done != nullptr) {
    __syncthreads();  // the flags of this block's wavefronts are on their way
    if (tid == 0) {
      __threadfence();
      const uint32_t before = __hip_atomic_fetch_add(blocks_done, 1u, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
      if (before + 1 == gridDim.x) {
        make_plan(varying, plan, rq);
      }
    }
  }
}

// What the scatter passes leave undone: nothing ran (all keys of every row are equal: the
// output is the input, the indices are 0..seg-1), or a single pass sorted in place into
// scratch buffer 1 and its result still has to reach the caller's array.
template <typename KeyT>
__global__ __launch_bounds__(256) void finalize_kernel(const SortPlan* __restrict__ plan,
                                                        const KeyT* in,
                                                        KeyT* out,
                                                        const KeyT* __restrict__ t1,
                                                        int64_t* __restrict__ idx_out,
                                                        uint64_t volume,
                                                        uint64_t seg,
                                                        int64_t index_offset,
                                                        PlanRequest rq)
{
  const uint32_t k      = plan->n_active;
  const uint64_t stride = static_cast<uint64_t>(gridDim.x) * blockDim.x;
  const uint64_t first  = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (k == 0) {
    if (rq.want_values && !rq.in_place) {
      for (uint64_t i = first; i < volume; i += stride) {
        out[i] = in[i];
      }
    }
    if (rq.want_indices) {
      for (uint64_t i = first; i < volume; i += stride) {
        idx_out[i] = static_cast<int64_t>(i % seg) + index_offset;
      }
    }
  } else if (k == 1 && rq.want_values && rq.in_place) {
    for (uint64_t i = first; i < volume; i += stride) {
      out[i] = t1[i];
    }
  }
}

// ---------------------------------------------------------------------------------------
// onesweep scatter pass
// ---------------------------------------------------------------------------------------
template <bool BIG>
struct SweepArgs {
  using OffT = typename RowWidth<BIG>::off_t;
  const void* key_buf[4];  // indexed by KeyBuf
  void* idx_buf[4];        // indexed by IdxBuf
  const SortPlan* plan;
  // resolved from the plan by the kernel before the tile is worked on:
  const void* keys_in;     // KeyT[volume]
  void* keys_out;          // KeyT[volume] or nullptr (last pass of an index-only sort)
  const OffT* idx_in;      // row positions from the previous pass, nullptr = synthesise
  void* idx_out;           // OffT[volume], or int64[volume] when idx_final
  int first;               // first running pass (ordered-key mode transforms the keys there)
  uint32_t* ticket;        // tile ticket counter of this pass (zeroed)
  uint32_t* xcd_tickets;   // XCD_COUNT tile counters of this pass (zeroed), see claim_tile
  const OffT* hist_excl;   // this pass's scanned histogram of row 0; row stride = hist_row_stride
  OffT* desc;              // [num_tiles][256] descriptors of this pass (zeroed)
  uint32_t* status;        // device status word
  uint64_t seg;            // row length
  uint64_t hist_row_stride;
  int64_t index_offset;
  uint32_t tiles_per_row;
  uint32_t num_tiles;
  int pass;                // which 8-bit digit this pass sorts by
  int idx_final;           // idx_out is the caller's int64 array
  uint32_t spin_limit;     // polls of one descriptor before the tile gives up (LOOKBACK_SPIN_LIMIT)
  uint32_t single_ticket;  // hand tiles out through `ticket` alone instead of the per-XCD counters
  const VirtPlan* vplan;   // virtual digits (virtual_digits.h), nullptr when the request cannot use them
  const DistinctTable* dtable;  // with vplan: the row's different keys when there are at most 256
  int free_rank;                // from the plan: this pass need not be stable
  // Index-only requests that may run on the ranks of the row's different keys: that one pass, when it
  // is to run, has been done by a launch of its own in a shape that stages one byte per key (DONLY
  // below), and the launch of the pass itself has nothing left to do.
  uint32_t distinct_pass_done;
};

// ---- which tile a workgroup takes ----
// The runs that neighbouring tiles write for one digit meet inside a 128-byte line (a run is 64
// elements on average and starts wherever the previous tile's run ended).  The two partial
// writes of such a line merge in an L2 only when both tiles run on the same XCD; from different
// XCDs they reach memory as two masked writes, which a store-pattern probe on this device prices
// at 1.10 ms against 0.79 ms for two 4-byte streams in runs of 61 elements (0.64 ms when the runs
// are whole lines).  So tiles are dealt in groups of TILE_GROUP consecutive tiles: group g
// belongs to XCD g % 8, and the workgroups of an XCD take the tiles of its groups in ascending
// order through a counter of their own.  A workgroup whose XCD has run out of tiles takes from
// the next XCD's groups, so every tile is taken exactly once whatever the dispatcher does, and
// the tiles below any taken tile of an XCD's own sequence are always taken too: a tile that a
// look-back waits for is either held by a resident workgroup or next in line on an XCD whose
// resident workgroups hold lower tiles only, which finish without it.  What the order does
// assume is that every XCD keeps receiving workgroups of this launch: if other work kept one XCD
// fully occupied for seconds, tiles elsewhere would wait for that XCD's share until the bounded
// look-back gave up and the call reported CPN_ERR_DEVICE.  A single counter for all XCDs has no
// such dependence, at the price of the split lines: cpn_set_tile_order selects it at run time
// (SweepArgs::single_ticket), and a caller that met CPN_ERR_DEVICE can repeat the sort that way.
constexpr uint32_t XCD_COUNT = 8;
#ifndef CPN_TILE_GROUP
#define CPN_TILE_GROUP 8
#endif
constexpr uint32_t TILE_GROUP = CPN_TILE_GROUP;

__device__ __forceinline__ uint32_t xcd_of_this_workgroup()
{
  uint32_t v;
  asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID, 0, 4)" : "=s"(v));
  return v & (XCD_COUNT - 1);
}

// Returns the tile for this workgroup, or 0xFFFFFFFF when every tile has been taken.
__device__ __forceinline__ uint32_t claim_tile(uint32_t* xcd_tickets, uint32_t num_tiles)
{
  const uint32_t groups = (num_tiles + TILE_GROUP - 1) / TILE_GROUP;
  const uint32_t home   = xcd_of_this_workgroup();
  for (uint32_t s = 0; s < XCD_COUNT; ++s) {
    const uint32_t y    = (home + s) & (XCD_COUNT - 1);
    const uint32_t mine = (groups > y) ? (groups - y + XCD_COUNT - 1) / XCD_COUNT : 0u;  // groups y, y+8, ...
    while (true) {
      const uint32_t n = __hip_atomic_fetch_add(xcd_tickets + y, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      const uint32_t m = n / TILE_GROUP;
      if (m >= mine) {
        break;  // this XCD's groups are used up: on to the next one's
      }
      const uint32_t tile = (m * XCD_COUNT + y) * TILE_GROUP + n % TILE_GROUP;
      if (tile < num_tiles) {
        return tile;
      }
      // (the last group of the sort may be short: take again)
    }
  }
  return 0xFFFFFFFFu;
}

#ifndef CPN_ONESWEEP_WAVES_PER_EU
#define CPN_ONESWEEP_WAVES_PER_EU 4
#endif

// Bytes per key of the LDS staging area: the wider of key and row position; DONLY kernels stage one
// byte per key (its digit) and the row positions.
template <typename KeyT, typename OffT, bool HAS_IDX, bool DONLY>
__host__ __device__ constexpr int sweep_stage_elem()
{
  return DONLY ? static_cast<int>(sizeof(OffT))
               : ((HAS_IDX && sizeof(OffT) > sizeof(KeyT)) ? static_cast<int>(sizeof(OffT)) : static_cast<int>(sizeof(KeyT)));
}

// Shared-memory view of one onesweep workgroup.
template <typename KeyT, typename OffT, int WAVES, int TILE, int STAGE_ELEM>
struct SweepShared {
  alignas(16) unsigned char stage[TILE * STAGE_ELEM];  // sorted tile: keys, then the payload
  uint32_t ctr[WAVES * RADIX];                         // per wave and digit: count, then first position
  OffT gbase[RADIX];                                   // per digit: row offset of sorted position 0
  uint32_t wsum[RADIX / WAVE];
  uint32_t tile;
};

// The work on one tile.  FULL is true for tiles of exactly TILE keys: every bounds test
// folds away and the body is straight-line code, which lets the compiler batch the LDS and
// HBM accesses of a phase instead of waiting on each one.
//
// XFORM (index-only sorts): the first running pass replaces the keys by their order-preserving
// unsigned image as soon as they are loaded and writes them out that way; every pass extracts
// digits with the identity codec, so the key transform is paid once per key instead of twice
// per pass.  The values themselves are never returned in that case.
//
// DONLY (with VIRT and HAS_IDX): the pass stores no keys (the one pass of an index-only sort on the
// ranks of the row's different keys); the keys are turned into digits as they arrive and only
// the digits, one byte each, go through LDS.
//
// UNFLIP (with XFORM, keys-only sorts of float keys that hold no NaN and no -0.0, SortPlan::flipped):
// the images that the first pass stored are mapped back to the keys' bits by the last pass as it
// stores them.
template <typename KeyT, int CODEC, bool XFORM, bool BIG, bool HAS_IDX, int BLOCK, int ITEMS, bool FULL, bool VIRT,
          bool DONLY = false, bool UNFLIP = false>
__device__ __forceinline__ void onesweep_tile(
  const SweepArgs<BIG>& a,
  const uint32_t vcount,    // VIRT: positions in this pass's group, their bit offsets (8 bits each)
  const uint64_t voffsets,  //       and their shifted lookup tables in LDS (virtual_digits.h)
  const uint8_t* vlut,
  SweepShared<KeyT, typename RowWidth<BIG>::off_t, BLOCK / WAVE, BLOCK * ITEMS,
              sweep_stage_elem<KeyT, typename RowWidth<BIG>::off_t, HAS_IDX, DONLY>()>& sh,
  const uint32_t tile,
  const uint64_t row,
  const uint32_t trow,
  const uint32_t count)
{
  using OffT = typename RowWidth<BIG>::off_t;
  using DB   = DescBits<OffT>;
  constexpr int WAVES = BLOCK / WAVE;
  constexpr int TILE  = BLOCK * ITEMS;
  constexpr int WTILE = ITEMS * WAVE;  // keys of one wave, contiguous in the tile
  constexpr int DCODEC = XFORM ? static_cast<int>(CODEC_UNSIGNED) : CODEC;  // codec at digit extraction

  const int tid           = threadIdx.x;
  const int lane          = tid & (WAVE - 1);
  const int wave          = tid / WAVE;
  const uint32_t woff     = wave * WTILE + lane;
  const uint64_t row_base = row * a.seg;
  const uint64_t tile_off = static_cast<uint64_t>(trow) * TILE;
  uint32_t* wctr          = sh.ctr + wave * RADIX;
  KeyT* s_keys            = reinterpret_cast<KeyT*>(sh.stage);
  OffT* s_idx             = reinterpret_cast<OffT*>(sh.stage);

  // ---- load: item i of lane l is element  wave*WTILE + i*64 + l  of the tile ----
  const KeyT* kin = static_cast<const KeyT*>(a.keys_in) + row_base + tile_off;
  // (DONLY: the keys are not kept; they arrive in groups of KEY_GROUP rounds, one group ahead of the
  // ranking, see below)
  constexpr int KEY_GROUP = 8;
  KeyT key[DONLY ? KEY_GROUP : ITEMS];
  auto load_key = [&](int i) -> KeyT {
    const uint32_t o = woff + i * WAVE;
    return (FULL || o < count) ? kin[o] : KeyT{};
  };
#pragma unroll
  for (int i = 0; i < (DONLY ? KEY_GROUP : ITEMS); ++i) {
    key[i] = load_key(i);
  }
  if constexpr (XFORM) {
    static_assert(!UNFLIP || (CODEC == CODEC_FLOAT && !HAS_IDX), "images are mapped back for keys-only float sorts");
    if (a.first) {  // one uniform branch around all items, so that the loads above stay batched
#pragma unroll
      for (int i = 0; i < ITEMS; ++i) {
        // (UNFLIP: no key is a NaN or a -0.0, for which alone the two images differ)
        key[i] = UNFLIP ? sign_flip<KeyT>(key[i]) : ordered_bits<CODEC, KeyT>(key[i]);
      }
    }
  }

  // ---- rank inside the wave (counters run from zero), count digits per wave ----
  // Sorts that return keys only: the first pass to run need not be stable (keys that tie in
  // every digit are the same bits, unless float keys hold a NaN or a -0.0, which the histogram
  // sweep has looked for; complex keys are left out; every later pass is stable), so its ranks
  // come from one LDS atomic per key on the counters of wave 0, which then serve the whole tile.
  constexpr bool FREE_FIRST_OK =
    !HAS_IDX && !VIRT && (CODEC == CODEC_UNSIGNED || CODEC == CODEC_SIGNED || CODEC == CODEC_FLOAT);
  const bool free_first = FREE_FIRST_OK && (a.free_rank != 0);
  const uint32_t* rank_base    = free_first ? sh.ctr : wctr;
  uint32_t dpk[ITEMS / 4];   // the digits, four per register
  uint32_t rnk2[ITEMS / 2];  // rank among the wave's keys of the same digit, two per register
  auto rank_item = [&](const int i, const KeyT k) {
    const bool valid = FULL || (woff + i * WAVE < count);
    uint32_t d;
    if constexpr (DONLY) {
      uint64_t ow[KeyTraits<DCODEC, KeyT>::NWORDS];
      KeyTraits<DCODEC, KeyT>::words(k, ow);
      d = distinct_rank(ow[0], reinterpret_cast<const uint64_t*>(vlut), vlut + DISTINCT_LOOKUP * 8);
    } else if constexpr (VIRT) {
      uint64_t ow[KeyTraits<DCODEC, KeyT>::NWORDS];
      KeyTraits<DCODEC, KeyT>::words(k, ow);
      d = virtual_digit(ow[0], vcount, voffsets, vlut);
    } else {
      d = KeyTraits<DCODEC, KeyT>::digit(k, a.pass);
    }
    dpk[i / 4]       = (i % 4 == 0) ? d : (dpk[i / 4] | (d << (8 * (i % 4))));
    uint32_t r;
    if (FREE_FIRST_OK && free_first) {  // uniform
      r = valid ? atomicAdd(&sh.ctr[d], 1u) : 0u;
    } else {
      r = wave_match_rank(d, valid, wctr) & 0xFFFFu;
    }
    rnk2[i / 2]      = (i % 2 == 0) ? r : (rnk2[i / 2] | (r << 16));
    // the packed registers are opaque to the optimiser, which would otherwise keep every
    // digit and rank alive in a register of its own until the scatter phase
    asm volatile("" : "+v"(dpk[i / 4]), "+v"(rnk2[i / 2]));
  };
  if constexpr (DONLY) {
    // 32 eight-byte keys would take 64 registers: the loads of the next KEY_GROUP rounds are issued
    // before the current group is ranked, and a key is dropped as soon as its digit is known
    static_assert(ITEMS % KEY_GROUP == 0, "whole groups of rounds");
#pragma unroll
    for (int g = 0; g < ITEMS / KEY_GROUP; ++g) {
      KeyT ahead[KEY_GROUP];
#pragma unroll
      for (int j = 0; j < KEY_GROUP; ++j) {
        ahead[j] = (g + 1 < ITEMS / KEY_GROUP) ? load_key((g + 1) * KEY_GROUP + j) : KeyT{};
      }
#pragma unroll
      for (int j = 0; j < KEY_GROUP; ++j) {
        rank_item(g * KEY_GROUP + j, key[j]);
      }
#pragma unroll
      for (int j = 0; j < KEY_GROUP; ++j) {
        key[j] = ahead[j];
      }
    }
  } else {
#pragma unroll
    for (int i = 0; i < ITEMS; ++i) {
      rank_item(i, key[i]);
    }
  }
  __syncthreads();

  // ---- per digit: start of every wave's keys, tile total, publish, first look-back reads:
  //      the answers travel while the tile is scattered into LDS ----
  uint32_t dsum = 0, dincl = 0;
  OffT window[LOOKBACK_WINDOW];
  OffT* my_desc     = a.desc + static_cast<uint64_t>(tile) * RADIX + tid;
  const uint32_t t0 = tile - trow;  // first tile of the row, always published INCLUSIVE
  if (tid < RADIX) {
#pragma unroll
    for (int w = 0; w < WAVES; ++w) {
      const uint32_t c        = sh.ctr[w * RADIX + tid];
      sh.ctr[w * RADIX + tid] = dsum;
      dsum += c;
    }
    const OffT first = (trow == 0) ? DB::INCLUSIVE : DB::AGGREGATE;
    __hip_atomic_store(my_desc, static_cast<OffT>(first | dsum), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (trow != 0) {
#pragma unroll
      for (int j = 0; j < LOOKBACK_WINDOW; ++j) {
        // tiles before the row start are replaced by the row's first tile (the sum stops there)
        const uint32_t t = (tile - 1 >= t0 + j) ? tile - 1 - j : t0;
        window[j] = __hip_atomic_load(a.desc + static_cast<uint64_t>(t) * RADIX + tid, __ATOMIC_RELAXED,
                                      __HIP_MEMORY_SCOPE_AGENT);
      }
    }
    dincl = wave_inclusive_scan(dsum, lane);
    if (lane == WAVE - 1) {
      sh.wsum[wave] = dincl;
    }
  }
  __syncthreads();
  uint32_t dexcl = 0;  // start of this digit's keys in the sorted tile
  if (tid < RADIX) {
    dexcl = dincl - dsum;
    for (int w = 0; w < wave; ++w) {
      dexcl += sh.wsum[w];
    }
#pragma unroll
    for (int w = 0; w < WAVES; ++w) {
      sh.ctr[w * RADIX + tid] += dexcl;
    }
  }
  __syncthreads();

  // ---- scatter into LDS: counter = first position of this wave's keys with that digit ----
  // VIRT kernels, passes that store no keys (the last pass of an index-only sort): only the digits
  // travel, one byte each, and the table lookups for the second use of the digit fall away
  const bool digits_only = DONLY || (VIRT && (a.keys_out == nullptr));
  uint32_t pos2[ITEMS / 2];  // positions in the sorted tile, two per register
#pragma unroll
  for (int i = 0; i < ITEMS; ++i) {
    const uint32_t d   = (dpk[i / 4] >> (8 * (i % 4))) & 0xFFu;
    const uint32_t pos = (rank_base[d] + ((rnk2[i / 2] >> (16 * (i % 2))) & 0xFFFFu)) & 0xFFFFu;
    if (FULL || (woff + i * WAVE < count)) {
      if (VIRT && digits_only) {
        reinterpret_cast<uint8_t*>(s_keys)[pos] = static_cast<uint8_t>(d);
      } else if constexpr (!DONLY) {
        s_keys[pos] = key[i];
      }
    }
    pos2[i / 2] = (i % 2 == 0) ? pos : (pos2[i / 2] | (pos << 16));
  }

  // ---- decoupled look-back over the earlier tiles of this row ----
  // A descriptor written on another XCD is only visible through memory-side accesses, so
  // one poll costs a full memory round trip.  The first window of predecessors was requested
  // before the scatter phase; its answers are summed front to back until the first
  // inclusive one, further windows follow only if none was.
  if (tid < RADIX) {
    OffT before = 0;
    if (trow != 0) {
      uint32_t hi = tile - 1;  // nearest predecessor not yet accounted for
      bool done   = false;
      bool failed = false;
      while (true) {
#pragma unroll
        for (int j = 0; j < LOOKBACK_WINDOW; ++j) {
          if (!done) {
            OffT w = window[j];
            if ((w & DB::STATUS) == 0) {
              const uint32_t t = (hi >= t0 + j) ? hi - j : t0;
              const OffT* dp   = a.desc + static_cast<uint64_t>(t) * RADIX + tid;
              uint32_t spins   = 0;
              do {
                if (++spins >= a.spin_limit) {
                  failed = true;
                  break;
                }
                if ((spins & 255u) == 0 &&
                    __hip_atomic_load(a.status, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0) {
                  failed = true;  // another tile already gave up: drain quickly
                  break;
                }
                __builtin_amdgcn_s_sleep(4);
                w = __hip_atomic_load(dp, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
              } while ((w & DB::STATUS) == 0);
            }
            if (failed) {
              done = true;
            } else {
              before += (w & DB::VALUE);
              if ((w & DB::INCLUSIVE) != 0) {
                done = true;
              }
            }
          }
        }
        if (done) {
          break;
        }
        hi = (hi >= t0 + LOOKBACK_WINDOW) ? hi - LOOKBACK_WINDOW : t0;
#pragma unroll
        for (int j = 0; j < LOOKBACK_WINDOW; ++j) {
          const uint32_t t = (hi >= t0 + j) ? hi - j : t0;
          window[j] = __hip_atomic_load(a.desc + static_cast<uint64_t>(t) * RADIX + tid, __ATOMIC_RELAXED,
                                        __HIP_MEMORY_SCOPE_AGENT);
        }
      }
      if (failed) {
        __hip_atomic_fetch_or(a.status, DEVICE_ERR_LOOKBACK, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
      __hip_atomic_store(my_desc, static_cast<OffT>(DB::INCLUSIVE | (before + dsum)), __ATOMIC_RELAXED,
                         __HIP_MEMORY_SCOPE_AGENT);
    }
    // offset inside the row of local sorted position 0 for this digit (unsigned wrap is fine)
    sh.gbase[tid] = a.hist_excl[row * a.hist_row_stride + tid] + before - static_cast<OffT>(dexcl);
  }
  __syncthreads();

  // ---- coalesced runs from LDS to HBM: the element at sorted position p of the tile goes
  //      to row offset gbase[its digit] + p.  The digits of this thread's output positions
  //      are kept (four per register) for the payload, which goes the same way. ----
  uint32_t dq[ITEMS / 4];
  if (VIRT && digits_only) {
    const uint8_t* s_digits = reinterpret_cast<const uint8_t*>(s_keys);
#pragma unroll
    for (int k = 0; k < ITEMS; ++k) {
      const uint32_t p = tid + k * BLOCK;
      const uint32_t d = (FULL || p < count) ? s_digits[p] : 0u;
      dq[k / 4]        = (k % 4 == 0) ? d : (dq[k / 4] | (d << (8 * (k % 4))));
    }
  } else if constexpr (!DONLY) {
    KeyT kk[ITEMS];
#pragma unroll
    for (int k = 0; k < ITEMS; ++k) {
      const uint32_t p = tid + k * BLOCK;
      kk[k]            = (FULL || p < count) ? s_keys[p] : KeyT{};
    }
#pragma unroll
    for (int k = 0; k < ITEMS; ++k) {
      uint32_t d;
      if constexpr (VIRT) {
        uint64_t ow[KeyTraits<DCODEC, KeyT>::NWORDS];
        KeyTraits<DCODEC, KeyT>::words(kk[k], ow);
        d = virtual_digit(ow[0], vcount, voffsets, vlut);
      } else {
        d = KeyTraits<DCODEC, KeyT>::digit(kk[k], a.pass);
      }
      dq[k / 4]        = (k % 4 == 0) ? d : (dq[k / 4] | (d << (8 * (k % 4))));
    }
    if (a.keys_out != nullptr) {
      if constexpr (UNFLIP) {
        if (a.idx_final) {  // the last pass: the caller gets the keys' own bits back
#pragma unroll
          for (int k = 0; k < ITEMS; ++k) {
            kk[k] = sign_unflip<KeyT>(kk[k]);
          }
        }
      }
      KeyT* kout = static_cast<KeyT*>(a.keys_out) + row_base;
#pragma unroll
      for (int k = 0; k < ITEMS; ++k) {
        const uint32_t p = tid + k * BLOCK;
        if (FULL || p < count) {
          kout[sh.gbase[(dq[k / 4] >> (8 * (k % 4))) & 0xFFu] + p] = kk[k];
        }
      }
    }
  }
  if constexpr (HAS_IDX) {
    // row positions from the previous pass, or synthesised by the first pass
    OffT idx[ITEMS];
    if (a.idx_in != nullptr) {
      const OffT* iin = a.idx_in + row_base + tile_off;
#pragma unroll
      for (int i = 0; i < ITEMS; ++i) {
        const uint32_t o = woff + i * WAVE;
        idx[i]           = (FULL || o < count) ? iin[o] : static_cast<OffT>(0);
      }
    } else {
#pragma unroll
      for (int i = 0; i < ITEMS; ++i) {
        idx[i] = static_cast<OffT>(tile_off + woff + i * WAVE);
      }
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < ITEMS; ++i) {
      if (FULL || (woff + i * WAVE < count)) {
        s_idx[(pos2[i / 2] >> (16 * (i % 2))) & 0xFFFFu] = idx[i];
      }
    }
    __syncthreads();
    if (a.idx_final) {
      int64_t* iout = static_cast<int64_t*>(a.idx_out) + row_base;
#pragma unroll
      for (int k = 0; k < ITEMS; ++k) {
        const uint32_t p = tid + k * BLOCK;
        if (FULL || p < count) {
          iout[sh.gbase[(dq[k / 4] >> (8 * (k % 4))) & 0xFFu] + p] = static_cast<int64_t>(s_idx[p]) + a.index_offset;
        }
      }
    } else {
      OffT* iout = static_cast<OffT*>(a.idx_out) + row_base;
#pragma unroll
      for (int k = 0; k < ITEMS; ++k) {
        const uint32_t p = tid + k * BLOCK;
        if (FULL || p < count) {
          iout[sh.gbase[(dq[k / 4] >> (8 * (k % 4))) & 0xFFu] + p] = s_idx[p];
        }
      }
    }
  }
}

template <typename KeyT, int CODEC, bool XFORM, bool BIG, bool HAS_IDX, int BLOCK, int ITEMS, bool VIRT = false,
          bool DONLY = false>
__global__ __launch_bounds__(BLOCK) __attribute__((amdgpu_waves_per_eu(CPN_ONESWEEP_WAVES_PER_EU)))
void onesweep_kernel(const SweepArgs<BIG> a_in)
{
  static_assert(!VIRT || (KeyTraits<CODEC, KeyT>::NWORDS == 1 && sizeof(KeyT) <= 8), "virtual digits: one ordered word");
  static_assert(!DONLY || (VIRT && HAS_IDX && !XFORM), "digits-only kernels: the index-only pass on the ranks of the different keys");
  // VIRT kernels can do both: the device-side plan says whether this sort runs on virtual digits
  bool virt_on = false;
  if constexpr (VIRT) {
    virt_on = (a_in.vplan != nullptr) && (a_in.vplan->enabled != VIRT_OFF);
  }
  using OffT = typename RowWidth<BIG>::off_t;
  static_assert(BLOCK >= RADIX, "one thread per digit is needed for the look-back");
  static_assert(ITEMS % 4 == 0, "digits are cached four to a register");
  constexpr int WAVES      = BLOCK / WAVE;
  constexpr int TILE       = BLOCK * ITEMS;
  constexpr int STAGE_ELEM = sweep_stage_elem<KeyT, OffT, HAS_IDX, DONLY>();
  static_assert(TILE <= 65536, "positions inside a tile are kept in 16 bits");

  __shared__ SweepShared<KeyT, OffT, WAVES, TILE, STAGE_ELEM> sh;
  __shared__ __align__(8) uint8_t s_vlut[VIRT ? VIRT_LDS_BYTES : 1];
  uint32_t vcount   = 0;
  uint64_t voffsets = 0;

  const PassPlan pp = a_in.plan->pass[a_in.pass];
  if (pp.active == 0) {
    return;  // every key of every row has the same digit here
  }
  if constexpr (VIRT) {
    // the index-only pass on the ranks of the row's different keys belongs to the DONLY launch,
    // where the request has one (distinct_pass_done), and everything else does not
    const bool its_pass = virt_on && a_in.vplan->enabled == VIRT_DISTINCT && pp.key_dst == BUF_NONE;
    if (DONLY ? !its_pass : (its_pass && a_in.distinct_pass_done != 0)) {
      return;
    }
  }
  if (VIRT && virt_on && a_in.vplan->enabled == VIRT_DISTINCT) {
    // the one pass on the ranks of the row's different keys: their lookup table into LDS
    vcount                 = VIRT_COUNT_DISTINCT;
    const DistinctTable* t = a_in.dtable;
    uint64_t* lk           = reinterpret_cast<uint64_t*>(s_vlut);
    for (uint32_t j = threadIdx.x; j < DISTINCT_LOOKUP; j += BLOCK) {
      lk[j]                           = t->lookup_keys[j];
      s_vlut[DISTINCT_LOOKUP * 8 + j] = t->lookup_rank[j];
    }
  } else if (VIRT && virt_on) {
    // this pass's group: the tables of its byte positions, codes shifted into place (made visible
    // by the barrier below), and the bit offsets of the bytes
    const VirtGroup& g = a_in.vplan->group[a_in.pass];
    vcount             = g.count;
    for (uint32_t j = 0; j < vcount; ++j) {
      voffsets |= static_cast<uint64_t>(g.pos[j] * RADIX_BITS) << (8 * j);
    }
    for (uint32_t j = threadIdx.x; j < vcount * RADIX; j += BLOCK) {
      const uint32_t which = j / RADIX;
      s_vlut[j] = static_cast<uint8_t>(a_in.vplan->lut[g.pos[which]][j % RADIX] << g.shift[which]);
    }
  }
  SweepArgs<BIG> a = a_in;
  a.keys_in        = a_in.key_buf[pp.key_src];
  a.keys_out       = (pp.key_dst == BUF_NONE) ? nullptr : const_cast<void*>(a_in.key_buf[pp.key_dst]);
  a.idx_in         = (pp.idx_src == BUF_NONE) ? nullptr : static_cast<const OffT*>(a_in.idx_buf[pp.idx_src]);
  a.idx_out        = a_in.idx_buf[pp.idx_dst];
  a.idx_final      = (pp.idx_dst == IDX_FINAL) ? 1 : 0;
  a.first          = static_cast<int>(pp.first & PLAN_FIRST);
  a.free_rank      = static_cast<int>((pp.first & PLAN_FREE_RANK) != 0);

  const int tid = threadIdx.x;
  // Tiles are handed out to the workgroups that are actually running, in ascending order per
  // XCD (claim_tile), so a tile that a look-back waits for is never stuck behind workgroups
  // that wait themselves.
  if (tid == 0) {
    // Once a tile of an earlier pass has given up, the keys in flight no longer match the
    // histograms the offsets come from, and a pass working on them could write past a row:
    // nothing more is sorted then.  (An ordinary load: what earlier launches wrote is visible
    // at the start of this one.  A failure inside this pass leaves its input consistent, every
    // offset stays inside the row, and waiting tiles notice the status word and drain.)
    uint32_t ticket;
    if (a.single_ticket != 0) {  // tiles in launch-wide ascending order, whichever XCD asks
      ticket = __hip_atomic_fetch_add(a.ticket, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (ticket >= a.num_tiles) {
        ticket = 0xFFFFFFFFu;
      }
    } else {
      ticket = claim_tile(a.xcd_tickets, a.num_tiles);
    }
    const uint32_t failed = *a.status;
    sh.tile               = (failed != 0) ? 0xFFFFFFFFu : ticket;
  }
  for (int j = tid; j < WAVES * RADIX; j += BLOCK) {
    sh.ctr[j] = 0;
  }
  __syncthreads();
  const uint32_t tile = sh.tile;
  if (tile >= a.num_tiles) {
    return;  // uniform per block: the sort has failed, see above (grid == num_tiles otherwise)
  }
  const uint64_t row    = tile / a.tiles_per_row;
  const uint32_t trow   = tile - static_cast<uint32_t>(row * a.tiles_per_row);
  const uint64_t remain = a.seg - static_cast<uint64_t>(trow) * TILE;
  if (VIRT && virt_on) {  // uniform for the launch
    if (remain >= static_cast<uint64_t>(TILE)) {
      onesweep_tile<KeyT, CODEC, XFORM, BIG, HAS_IDX, BLOCK, ITEMS, true, VIRT, DONLY>(a, vcount, voffsets, s_vlut, sh, tile,
                                                                                      row, trow, TILE);
    } else {
      onesweep_tile<KeyT, CODEC, XFORM, BIG, HAS_IDX, BLOCK, ITEMS, false, VIRT, DONLY>(a, vcount, voffsets, s_vlut, sh, tile,
                                                                                       row, trow, static_cast<uint32_t>(remain));
    }
    return;
  }
  // keys-only sorts of float keys: the device-side plan says whether the passes run on stored images
  // (keys of 4 and 8 bytes: the transform of a 2-byte key is cheap, and the second code path costs its
  // kernel a workgroup per CU)
  constexpr bool CAN_FLIP = !HAS_IDX && !XFORM && !DONLY && CODEC == CODEC_FLOAT && KeyTraits<CODEC, KeyT>::NWORDS == 1 &&
                            sizeof(KeyT) >= 4;
  if constexpr (CAN_FLIP) {
    if (a_in.plan->flipped != 0) {  // uniform for the sort
      if (remain >= static_cast<uint64_t>(TILE)) {
        onesweep_tile<KeyT, CODEC, true, BIG, HAS_IDX, BLOCK, ITEMS, true, false, false, true>(a, 0u, 0ull, nullptr, sh, tile,
                                                                                                row, trow, TILE);
      } else {
        onesweep_tile<KeyT, CODEC, true, BIG, HAS_IDX, BLOCK, ITEMS, false, false, false, true>(
          a, 0u, 0ull, nullptr, sh, tile, row, trow, static_cast<uint32_t>(remain));
      }
      return;
    }
  }
  if constexpr (!DONLY) {  // (a DONLY launch has returned above unless the virtual plan is in force)
    if (remain >= static_cast<uint64_t>(TILE)) {
      onesweep_tile<KeyT, CODEC, XFORM, BIG, HAS_IDX, BLOCK, ITEMS, true, false>(a, 0u, 0ull, nullptr, sh, tile, row, trow, TILE);
    } else {
      onesweep_tile<KeyT, CODEC, XFORM, BIG, HAS_IDX, BLOCK, ITEMS, false, false>(a, 0u, 0ull, nullptr, sh, tile, row, trow,
                                                                                  static_cast<uint32_t>(remain));
    }
  }
}

}  // namespace cpn
