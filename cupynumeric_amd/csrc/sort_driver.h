// Host side of the sort: path choice, workspace layout, buffer ping-pong and launches.
//
// Plays the role of cub_local_sort / thrust_local_sort and their temporary-buffer handling
// (src/cupynumeric/sort/cub_sort.cuh:36-193, src/cupynumeric/sort/thrust_sort.cuh:37-124),
// with the workspace supplied by the caller instead of a Legate pool.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/cpn_sort.h"
#include "count_row_sort.h"
#include "lds_row_sort.h"
#include "onesweep.h"
#include "profile.h"
#include "tiny_row_sort.h"
#include "bitonic_row_sort.h"
#include "merge_rows.h"
#include "wave_row_sort.h"

namespace cpn {

// Set by HIP_TRY when a runtime call fails; read through cpn_last_hip_error().
extern thread_local int g_last_hip_error;

#define CPN_HIP_TRY(expr)                        \
  do {                                           \
    const hipError_t cpn_err_ = (expr);          \
    if (cpn_err_ != hipSuccess) {                \
      ::cpn::g_last_hip_error = (int)cpn_err_;   \
      (void)hipGetLastError();                   \
      return CPN_ERR_HIP;                        \
    }                                            \
  } while (0)

constexpr uint64_t WORKSPACE_ALIGN  = 256;
// Workspace header: [0] status word, [128..) tile tickets, [256..) per-pass "digit varies" flags,
// [384..) the device-side SortPlan.  The status word has a 128-byte line to itself: every tile
// reads it with an ordinary load, and the tickets next door are under constant atomic traffic.
constexpr uint64_t HEADER_BYTES     = 2048;
constexpr uint64_t HEADER_TICKETS   = 128;
constexpr uint64_t HEADER_SCAN_DONE = 240;  // blocks of the scan kernel that have finished
constexpr uint64_t HEADER_SPECIALS  = 244;  // float keys: the sort holds a NaN or a -0.0
constexpr uint64_t HEADER_VARYING   = 256;
constexpr uint64_t HEADER_PLAN      = 384;
constexpr uint64_t HEADER_XCD_TICKETS = 1024;  // per pass: one tile counter per XCD (onesweep.h, claim_tile)
static_assert(HEADER_TICKETS + 4 * MAX_PASSES <= HEADER_SCAN_DONE, "tickets overlap the scan counter");
static_assert(HEADER_VARYING + 4 * MAX_PASSES <= HEADER_PLAN, "flags overlap the plan");
static_assert(HEADER_PLAN + sizeof(SortPlan) <= HEADER_XCD_TICKETS, "plan overlaps the per-XCD tile counters");
static_assert(HEADER_XCD_TICKETS + 4 * XCD_COUNT * MAX_PASSES <= HEADER_BYTES, "tile counters do not fit the header");
constexpr uint64_t BIG_ROW_ELEMENTS = 1ull << 30;
// Shortest row for which virtual digits are considered: their extra launches (three small kernels
// and an early-exiting twin of every pass) cost about 0.1 ms, 2 % of a 2^26-key sort of 8-byte keys.
constexpr uint64_t VIRT_MIN_ROW_ELEMENTS = 1ull << 26;
// The threshold in force (cpn_set_virtual_digit_threshold; tests lower it).
uint64_t virtual_digit_threshold();
// How the scatter passes hand out their tiles: per XCD (default) or through one counter
// (cpn_set_tile_order, CPN_SORT_TILE_ORDER=single).
bool tile_order_single();
// Rows of at least this many elements use 64-bit counts, descriptors and row positions:
// BIG_ROW_ELEMENTS unless lowered by cpn_set_wide_row_threshold / CPN_SORT_WIDE_ROW_THRESHOLD
// (for tests that exercise the 64-bit kernels without a 2^30-element row).
uint64_t wide_row_threshold();

__host__ __device__ constexpr uint64_t align_up(uint64_t v, uint64_t a) { return (v + a - 1) / a * a; }

// Tile shape of the global sort per key width (the macros allow A/B builds of other shapes).
#ifndef CPN_GLOBAL_BLOCK
#define CPN_GLOBAL_BLOCK 512
#endif
#ifndef CPN_GLOBAL_ITEMS
#define CPN_GLOBAL_ITEMS 32
#endif
// 8-byte keys: 1024 threads x 16 keys, one workgroup per CU (144 KiB of LDS), so that a tile is
// 16 384 keys like the tiles of 4-byte keys and a digit's run 64 keys on average.  Measured on 2^27
// keys against 512 threads (8192-key tiles, two workgroups per CU): float64 sort 5.24 -> 5.02 ms,
// argsort 6.51 -> 6.16, int64 sort 5.04 -> 4.67; the one pass of a row of 16 different int64 keys
// 0.66 -> 0.71 ms.  16-byte keys likewise (1024 x 8 keys: 2^25 complex128 keys 4.91 -> 4.69 ms).
// 4-byte keys: 512 threads x 32 keys (1024 threads: 3.94 -> 4.33 ms at 2^28).
__host__ __device__ constexpr int global_block(int key_bytes) { return key_bytes >= 8 ? 1024 : CPN_GLOBAL_BLOCK; }
// (64-bit keys or 64-bit row positions halve the items per thread: the LDS staging area stays at
// 64 KiB for 512 threads, two workgroups per CU, and is 128 KiB for the 1024 threads of 8-byte keys)
__host__ __device__ constexpr int global_items(int key_bytes, bool big)
{
  return key_bytes == 16 ? 8 : ((key_bytes == 8 || big) ? 16 : CPN_GLOBAL_ITEMS);
}
__host__ __device__ constexpr int global_tile(int key_bytes, bool big)
{
  return global_block(key_bytes) * global_items(key_bytes, big);
}

// Longest row the LDS kernel can take, per key width: 1024 threads with the row, the staged row
// positions of an argsort (2 bytes each) and 16 KiB of per-wave digit counters in the CU's 160 KiB
// of LDS.  Keys of up to 4 bytes: 16 per thread (64 + 32 + 16 KiB).  8-byte keys: 16 per thread for
// values only (128 + 16 KiB), 14 with positions (112 + 28 + 16 KiB).  16-byte keys: 4 per thread.
__host__ __device__ constexpr uint64_t lds_row_capacity(int key_bytes, bool with_positions)
{
  return key_bytes == 16 ? 4096 : (key_bytes == 8 ? (with_positions ? 14336 : 16384) : 16384);
}
// Values-only sorts of 2-byte keys: the counting kernel (count_row_sort.h) needs no room for the row beside
// its 65 536 bins and takes rows of up to 57 344 keys (lds_row_limit says whether it is in use).
constexpr uint64_t COUNT16_ROW_CAPACITY = 57344;
// Radix passes of a key: one per byte, plus the NaN-class pass of complex keys.
__host__ __device__ constexpr int key_passes(int key_bytes, int codec)
{
  return codec == CODEC_COMPLEX ? key_bytes + 1 : key_bytes;
}

// Short rows of real keys (2 ... bitonic_row_limit keys) go through the sorting network (bitonic_row_sort.h)
// unless CPN_SORT_BITONIC_ROWS=0 in the environment sends them to the ranking kernels (A/B runs).
bool bitonic_rows_enabled();
// Longest row that goes through the network, per key width and with or without positions; the environment
// variable CPN_SORT_BITONIC_ROW_LIMIT lowers it (A/B runs).
uint64_t bitonic_row_limit(int key_bytes, bool with_positions, bool float_keys);

// Row length up to which one wavefront (instead of one workgroup) sorts a row; at most 1024.
// Changed by cpn_set_wave_row_limit / CPN_SORT_WAVE_ROW_LIMIT for A/B runs.
uint64_t wave_row_limit();

// Shortest row of 2-byte keys that a values-only sort gives to the counting kernel
// (count_row_sort.h): COUNT16_MIN_ROW unless CPN_SORT_COUNT16_MIN_ROW in the environment says
// otherwise (A/B runs; a value above the LDS row capacity switches the kernel off).
uint64_t count16_min_row();

// Row length up to which the LDS kernel is used.  Equals lds_row_capacity unless the
// environment variable CPN_SORT_LDS_ROW_LIMIT or cpn_set_lds_row_limit lowers it, e.g. to 0
// to send every request down the global path for an A/B run.
uint64_t lds_row_limit(int key_bytes, bool with_positions);

// Rows longer than the per-row kernels take: cut into 2^levels pieces that the per-row kernel sorts,
// merged pairwise level by level (merge_rows.h) instead of going down the global path.  Real keys
// of 4 and 8 bytes.  Off when cpn_set_merge_rows(0) / CPN_SORT_MERGE_ROWS=0 says so, and whenever
// the LDS row limit has been lowered (an A/B run that wants the global path gets it).
// merge_levels_limit: the most levels for which this beats the global path, whose cost is one pass
// per key byte whatever the row length, while every level here is one read and one write of the rows.
bool merge_rows_enabled();
int merge_levels_limit(int key_bytes, bool want_indices);
// Levels of merging for rows of seg elements: 0 = the request does not take this path.
inline int merged_row_levels(int key_bytes, int passes, uint64_t volume, uint64_t seg, bool want_indices)
{
  if (!merge_rows_enabled() || (key_bytes != 4 && key_bytes != 8) || passes != key_bytes || volume == 0) {
    return 0;
  }
  const uint64_t cap = lds_row_capacity(key_bytes, want_indices);
  if (lds_row_limit(key_bytes, want_indices) != cap || seg <= cap || seg >= (1ull << 31)) {
    return 0;  // (the merge kernels count inside a row in 32 bits)
  }
  const int limit = merge_levels_limit(key_bytes, want_indices);
  int levels      = 1;
  while ((cap << levels) < seg) {
    if (++levels > limit) {
      return 0;
    }
  }
  if (levels > limit) {
    return 0;
  }
  // one workgroup of a merge per chunk of a pair of pieces, one of the per-row kernel per piece
  const uint64_t per_row = (seg + MERGE_CHUNK_MIN - 1) / MERGE_CHUNK_MIN + (1ull << levels);
  return (volume / seg) * per_row < (1ull << 31) ? levels : 0;
}
// Length of the pieces (the last one of a row may be shorter).
inline uint64_t merged_row_piece(uint64_t seg, int levels) { return (seg + (1ull << levels) - 1) >> levels; }
// Bytes of the table of chunk starts that a level of merging reads (one word per workgroup of the
// largest merge launch; every level reuses it).
inline uint64_t merged_row_split_bytes(uint64_t volume, uint64_t seg, int levels)
{
  const uint64_t per_row = (seg + MERGE_CHUNK_MIN - 1) / MERGE_CHUNK_MIN + (1ull << levels);
  return align_up((volume / seg) * per_row * sizeof(uint32_t), WORKSPACE_ALIGN);
}

// Element type code (enum cpn_dtype) -> key width and codec.
struct KeyKind {
  int bytes;  // 0 = unknown code
  int codec;  // -1 = known but unsupported
};

inline KeyKind key_kind(int dtype)
{
  switch (dtype) {
    case CPN_BOOL: return {1, CODEC_UNSIGNED};
    case CPN_INT8: return {1, CODEC_SIGNED};
    case CPN_INT16: return {2, CODEC_SIGNED};
    case CPN_INT32: return {4, CODEC_SIGNED};
    case CPN_INT64: return {8, CODEC_SIGNED};
    case CPN_UINT8: return {1, CODEC_UNSIGNED};
    case CPN_UINT16: return {2, CODEC_UNSIGNED};
    case CPN_UINT32: return {4, CODEC_UNSIGNED};
    case CPN_UINT64: return {8, CODEC_UNSIGNED};
    case CPN_FLOAT16: return {2, CODEC_FLOAT};
    case CPN_FLOAT32: return {4, CODEC_FLOAT};
    case CPN_FLOAT64: return {8, CODEC_FLOAT};
    case CPN_COMPLEX64: return {8, CODEC_COMPLEX};
    case CPN_COMPLEX128: return {16, CODEC_COMPLEX};
    default: return {0, -1};
  }
}

struct SortRequest {
  const void* values_in;
  void* values_out;      // may be nullptr
  int64_t* indices_out;  // may be nullptr
  uint64_t volume;
  uint64_t seg;
  int64_t index_offset;
  void* temp;
  uint64_t temp_bytes;
  hipStream_t stream;
  uint64_t row_stride = 0;  // elements between the starts of two rows, in input and outputs; 0: seg (dense rows)
  // Rows sorted piece by piece (and merged afterwards): every row is `pieces` pieces of seg elements,
  // the last one of last_seg; volume / seg still counts the rows.
  uint32_t pieces   = 1;
  uint32_t last_seg = 0;
  // CPN_SORT_SINGLE_TICKET of cpn_local_sort_ex: this call hands its tiles out through one counter,
  // whatever the process-wide tile order says
  bool single_ticket = false;
};

// Workspace layout of the global path.  Everything in [0, zero_bytes) is cleared per call.
struct GlobalLayout {
  bool big;
  bool virt;          // the request may use virtual digits (virtual_digits.h): a VirtPlan slot follows the header
  uint64_t off_virt;
  int passes;
  uint64_t rows;
  uint32_t tiles_per_row;
  uint64_t num_tiles;
  uint64_t off_hist, hist_bytes;
  uint64_t off_desc, desc_bytes_per_pass;
  uint64_t zero_bytes;
  uint64_t off_key1, off_key2, key_bytes_total;
  uint64_t off_idx, idx_bytes_total;
  uint64_t total;
  bool valid;
};

inline GlobalLayout global_layout(int key_bytes, int passes, uint64_t volume, uint64_t seg, bool want_values,
                                  bool want_indices, bool in_place)
{
  GlobalLayout L{};
  L.big           = seg >= wide_row_threshold();
  L.passes        = passes;
  L.rows          = volume / seg;
  const uint64_t tile = static_cast<uint64_t>(global_tile(key_bytes, L.big));
  const uint64_t tpr  = (seg + tile - 1) / tile;
  L.num_tiles         = tpr * L.rows;
  L.valid             = (tpr < (1ull << 32)) && (L.num_tiles < (1ull << 32));
  L.tiles_per_row     = static_cast<uint32_t>(tpr);
  const uint64_t ow   = L.big ? 8 : 4;
  // virtual digits: one long row of real 8-byte keys.  Their extra launches (three small kernels
  // and one early-exiting twin per pass, about 10 us each at this grid size) cost a 2^28-key sort
  // of 4-byte keys 2 %, more than four passes can win back on average; eight passes can.
  L.virt     = (L.rows == 1) && !L.big && (key_bytes == 8) && (passes == key_bytes) && (seg >= virtual_digit_threshold());
  L.off_virt = L.virt ? HEADER_BYTES : 0;
  L.off_hist          = HEADER_BYTES + (L.virt ? VIRT_WORKSPACE_BYTES : 0);
  L.hist_bytes        = align_up(L.rows * L.passes * RADIX * ow, WORKSPACE_ALIGN);
  L.off_desc          = L.off_hist + L.hist_bytes;
  L.desc_bytes_per_pass = align_up(L.num_tiles * RADIX * ow, WORKSPACE_ALIGN);
  L.zero_bytes        = L.off_desc + L.desc_bytes_per_pass * L.passes;
  uint64_t off        = L.zero_bytes;
  L.key_bytes_total   = align_up(volume * key_bytes, WORKSPACE_ALIGN);
  L.off_key1 = L.off_key2 = 0;
  bool need_key1, need_key2;
  // (see plan_kernel: intermediate passes alternate between buffer 1 and either the caller's
  // value array, when it is not also the input, or buffer 2)
  if (L.passes == 1) {
    need_key1 = want_values && in_place;
    need_key2 = false;
  } else {
    need_key1 = true;
    need_key2 = (!want_values || in_place) && L.passes >= 3;
  }
  if (need_key1) {
    L.off_key1 = off;
    off += L.key_bytes_total;
  }
  if (need_key2) {
    L.off_key2 = off;
    off += L.key_bytes_total;
  }
  L.off_idx         = 0;
  L.idx_bytes_total = align_up(volume * ow, WORKSPACE_ALIGN);
  if (want_indices && L.passes >= 2) {
    L.off_idx = off;
    off += L.idx_bytes_total;
  }
  L.total = off;
  return L;
}

inline uint64_t workspace_bytes(int key_bytes, int passes, uint64_t volume, uint64_t seg, bool want_values,
                                bool want_indices, bool in_place)
{
  if (volume == 0 || seg <= lds_row_limit(key_bytes, want_indices)) {
    return HEADER_BYTES;
  }
  if (const int levels = merged_row_levels(key_bytes, passes, volume, seg, want_indices); levels != 0) {
    // the rows with their pieces sorted: keys, and the int64 positions of an argsort; twice that
    // where the levels of merging go back and forth between two copies
    const uint64_t copy =
      align_up(volume * key_bytes, WORKSPACE_ALIGN) + (want_indices ? align_up(volume * 8, WORKSPACE_ALIGN) : 0);
    return HEADER_BYTES + merged_row_split_bytes(volume, seg, levels) + (levels >= 2 ? 2 : 1) * copy;
  }
  const GlobalLayout L = global_layout(key_bytes, passes, volume, seg, want_values, want_indices, in_place);
  return L.valid ? L.total : 0;
}

inline int launch_zero_fill(void* p, uint64_t bytes, hipStream_t stream)
{
  const uint64_t n_vec = bytes / 16;  // bytes is a multiple of 256
  uint64_t blocks      = (n_vec + 255) / 256;
  if (blocks > 4096) {
    blocks = 4096;
  }
  if (blocks == 0) {
    return CPN_OK;
  }
  {
    ProfileScope prof("zero_fill", stream);
    hipLaunchKernelGGL(zero_fill_kernel, dim3(static_cast<uint32_t>(blocks)), dim3(256), 0, stream,
                       static_cast<uint4*>(p), n_vec);
  }
  CPN_HIP_TRY(hipGetLastError());
  return CPN_OK;
}

// ---- rows longer than the LDS capacity: sorted pieces, merged pairwise --------------------------
template <typename KeyT, int CODEC, bool HAS_IDX>
inline int sort_rows_in_lds(const SortRequest& r);

template <typename KeyT, int CODEC, bool HAS_IDX>
int sort_rows_merged(const SortRequest& r, int levels)
{
  const uint64_t n = r.seg, rows = r.volume / n;
  const uint64_t q        = merged_row_piece(n, levels);
  const uint32_t pieces   = 1u << levels;  // (pieces - 1) * q < n: the last piece is never empty
  const uint64_t key_copy = align_up(r.volume * sizeof(KeyT), WORKSPACE_ALIGN);
  const uint64_t copy     = key_copy + (HAS_IDX ? align_up(r.volume * 8, WORKSPACE_ALIGN) : 0);
  uint32_t* splits        = reinterpret_cast<uint32_t*>(static_cast<uint8_t*>(r.temp) + HEADER_BYTES);
  uint8_t* ws             = static_cast<uint8_t*>(r.temp) + HEADER_BYTES + merged_row_split_bytes(r.volume, n, levels);
  // the copy that level `done` (0: the sorted pieces) leaves its rows in; the last level writes the outputs
  auto keys_of = [&](int done) { return reinterpret_cast<KeyT*>(ws + ((levels - 1 - done) % 2) * copy); };
  auto idx_of  = [&](int done) {
    return HAS_IDX ? reinterpret_cast<int64_t*>(ws + ((levels - 1 - done) % 2) * copy + key_copy) : nullptr;
  };
  {
    SortRequest c = r;
    c.values_out  = keys_of(0);
    c.indices_out = idx_of(0);
    c.seg         = q;
    c.volume      = rows * q;
    c.row_stride  = n;
    c.pieces      = pieces;
    c.last_seg    = static_cast<uint32_t>(n - (pieces - 1) * q);
    const int rc  = sort_rows_in_lds<KeyT, CODEC, HAS_IDX>(c);
    if (rc != CPN_OK) {
      return rc;
    }
  }
  for (int level = 1; level <= levels; ++level) {
    const uint64_t piece  = q << (level - 1);
    const uint32_t pairs  = pieces >> level;
    const uint64_t chunks = (2 * piece + merge_chunk(HAS_IDX) - 1) / merge_chunk(HAS_IDX);
    const bool last       = level == levels;
    const uint32_t grid   = static_cast<uint32_t>(rows * pairs * chunks);
    {
      ProfileScope prof("merge_split", r.stream);
      hipLaunchKernelGGL((merge_split_kernel<KeyT, CODEC>), dim3((grid + MERGE_SPLIT_BLOCK - 1) / MERGE_SPLIT_BLOCK),
                         dim3(MERGE_SPLIT_BLOCK), 0, r.stream, keys_of(level - 1), splits, static_cast<uint32_t>(n),
                         static_cast<uint32_t>(piece), static_cast<uint32_t>(chunks), pairs,
                         static_cast<uint32_t>(merge_chunk(HAS_IDX)), grid);
    }
    CPN_HIP_TRY(hipGetLastError());
    {
      ProfileScope prof("merge_halves", r.stream);
      hipLaunchKernelGGL((merge_halves_kernel<KeyT, CODEC, HAS_IDX>), dim3(grid), dim3(merge_block(HAS_IDX)), 0, r.stream,
                         keys_of(level - 1), idx_of(level - 1), last ? static_cast<KeyT*>(r.values_out) : keys_of(level),
                         last ? r.indices_out : idx_of(level), splits, static_cast<uint32_t>(n), static_cast<uint32_t>(piece),
                         static_cast<uint32_t>(chunks), pairs);
    }
    CPN_HIP_TRY(hipGetLastError());
  }
  return CPN_OK;
}

// ---- per-row LDS path ------------------------------------------------------------------
template <typename KeyT, int CODEC, bool HAS_IDX, int BLOCK, int ITEMS>
inline int launch_lds_rows(const SortRequest& r)
{
  const uint64_t rows = r.volume / r.seg;
  {
    ProfileScope prof("lds_row_sort", r.stream);
    hipLaunchKernelGGL((lds_row_sort_kernel<KeyT, CODEC, HAS_IDX, BLOCK, ITEMS>),
                       dim3(static_cast<uint32_t>(rows * r.pieces)), dim3(BLOCK), 0, r.stream,
                       static_cast<const KeyT*>(r.values_in), static_cast<KeyT*>(r.values_out), r.indices_out,
                       static_cast<uint32_t>(r.seg), r.row_stride != 0 ? r.row_stride : r.seg, r.pieces,
                       r.pieces > 1 ? r.last_seg : static_cast<uint32_t>(r.seg), r.index_offset,
                       static_cast<uint32_t*>(r.temp));
  }
  CPN_HIP_TRY(hipGetLastError());
  return CPN_OK;
}

// Compute units of the current device (the persistent grid of the counting kernel), looked up once.
inline int compute_units()
{
  static thread_local int cached_device = -1;
  static thread_local int cached_count  = 0;
  int dev                               = 0;
  if (hipGetDevice(&dev) != hipSuccess) {
    return 256;
  }
  if (dev != cached_device) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) {
      n = 256;
    }
    cached_device = dev;
    cached_count  = n;
  }
  return cached_count;
}

template <int CODEC>
inline int launch_count16_rows(const SortRequest& r)
{
  const uint64_t rows = r.volume / r.seg;
  {
    ProfileScope prof("count16_row_sort", r.stream);
    if (r.seg <= 8192) {
      const uint64_t cus  = static_cast<uint64_t>(compute_units());
      const uint64_t grid = rows < cus ? rows : cus;  // one workgroup per CU, each loops over its rows
      hipLaunchKernelGGL((count16_rows_kernel<CODEC>), dim3(static_cast<uint32_t>(grid)), dim3(COUNT16_BLOCK), 0, r.stream,
                         static_cast<const uint16_t*>(r.values_in), static_cast<uint16_t*>(r.values_out),
                         static_cast<uint32_t>(r.seg), static_cast<uint32_t>(rows), static_cast<uint32_t*>(r.temp));
    } else if (r.seg <= 16384) {
      hipLaunchKernelGGL((count16_long_rows_kernel<CODEC, 16>), dim3(static_cast<uint32_t>(rows)), dim3(COUNT16_BLOCK), 0,
                         r.stream, static_cast<const uint16_t*>(r.values_in), static_cast<uint16_t*>(r.values_out),
                         static_cast<uint32_t>(r.seg), static_cast<uint32_t*>(r.temp));
    } else if (r.seg <= 32768) {
      // 16 385 ... 32 768 keys: 32 keys per thread
      hipLaunchKernelGGL((count16_long_rows_kernel<CODEC, 32>), dim3(static_cast<uint32_t>(rows)), dim3(COUNT16_BLOCK), 0,
                         r.stream, static_cast<const uint16_t*>(r.values_in), static_cast<uint16_t*>(r.values_out),
                         static_cast<uint32_t>(r.seg), static_cast<uint32_t*>(r.temp));
    } else {
      // ... 57 344 keys: 56 keys per thread (counts and offsets of a row have to fit 16 bits)
      hipLaunchKernelGGL((count16_long_rows_kernel<CODEC, 56>), dim3(static_cast<uint32_t>(rows)), dim3(COUNT16_BLOCK), 0,
                         r.stream, static_cast<const uint16_t*>(r.values_in), static_cast<uint16_t*>(r.values_out),
                         static_cast<uint32_t>(r.seg), static_cast<uint32_t*>(r.temp));
    }
  }
  CPN_HIP_TRY(hipGetLastError());
  return CPN_OK;
}

template <typename KeyT, int CODEC, bool HAS_IDX, int ITEMS>
inline int launch_wave_rows(const SortRequest& r)
{
  constexpr int LDS_PER_ROW    = wave_row_lds_bytes<CODEC, KeyT, ITEMS, HAS_IDX>();
  constexpr int ROWS_PER_BLOCK = LDS_PER_ROW <= 12 * 1024 ? 4 : (LDS_PER_ROW <= 24 * 1024 ? 2 : 1);
  const uint64_t rows          = r.volume / r.seg;
  const uint64_t blocks        = (rows + ROWS_PER_BLOCK - 1) / ROWS_PER_BLOCK;
  {
    ProfileScope prof("wave_row_sort", r.stream);
    hipLaunchKernelGGL((wave_row_sort_kernel<KeyT, CODEC, HAS_IDX, ITEMS, ROWS_PER_BLOCK>),
                       dim3(static_cast<uint32_t>(blocks)), dim3(WAVE * ROWS_PER_BLOCK), 0, r.stream,
                       static_cast<const KeyT*>(r.values_in), static_cast<KeyT*>(r.values_out), r.indices_out,
                       static_cast<uint32_t>(r.seg), rows, r.index_offset, static_cast<uint32_t*>(r.temp));
  }
  CPN_HIP_TRY(hipGetLastError());
  return CPN_OK;
}

template <typename KeyT, int CODEC, bool HAS_IDX, int LANES, int E>
inline int launch_bitonic_rows(const SortRequest& r)
{
  const uint64_t rows           = r.volume / r.seg;
  const uint64_t rows_per_block = (256 / WAVE) * (WAVE / LANES);
  const uint64_t blocks         = (rows + rows_per_block - 1) / rows_per_block;
  {
    ProfileScope prof("bitonic_row_sort", r.stream);
    hipLaunchKernelGGL((bitonic_row_sort_kernel<KeyT, CODEC, HAS_IDX, LANES, E>), dim3(static_cast<uint32_t>(blocks)),
                       dim3(256), 0, r.stream, static_cast<const KeyT*>(r.values_in), static_cast<KeyT*>(r.values_out),
                       r.indices_out, static_cast<uint32_t>(r.seg), rows, r.index_offset, static_cast<uint32_t*>(r.temp));
  }
  CPN_HIP_TRY(hipGetLastError());
  return CPN_OK;
}
// A row of more than 4 LANES and up to 8 LANES keys: LANES lanes of 8 elements, or half as many lanes of 10, 12
// or 14 (fewer of the network's steps cross lanes), whichever covers the row.
template <typename KeyT, int CODEC, bool HAS_IDX, int LANES>
inline int launch_bitonic_lanes(const SortRequest& r)
{
  static_assert(LANES >= 2, "half the lanes");
  const uint64_t e = (r.seg + LANES - 1) / LANES;
  if (e <= 5) {
    return launch_bitonic_rows<KeyT, CODEC, HAS_IDX, LANES / 2, 10>(r);
  } else if (e == 6) {
    return launch_bitonic_rows<KeyT, CODEC, HAS_IDX, LANES / 2, 12>(r);
  } else if (e == 7) {
    return launch_bitonic_rows<KeyT, CODEC, HAS_IDX, LANES / 2, 14>(r);
  }
  return launch_bitonic_rows<KeyT, CODEC, HAS_IDX, LANES, 8>(r);
}

template <typename KeyT, int CODEC, bool HAS_IDX, int S>
inline int launch_tiny_rows(const SortRequest& r)
{
  const uint64_t rows          = r.volume / r.seg;
  const uint64_t rows_per_block = (256 / WAVE) * (WAVE / S);
  const uint64_t blocks        = (rows + rows_per_block - 1) / rows_per_block;
  {
    ProfileScope prof("tiny_row_sort", r.stream);
    hipLaunchKernelGGL((tiny_row_sort_kernel<KeyT, CODEC, HAS_IDX, S>), dim3(static_cast<uint32_t>(blocks)), dim3(256),
                       0, r.stream, static_cast<const KeyT*>(r.values_in), static_cast<KeyT*>(r.values_out),
                       r.indices_out, static_cast<uint32_t>(r.seg), rows, r.index_offset, static_cast<uint32_t*>(r.temp));
  }
  CPN_HIP_TRY(hipGetLastError());
  return CPN_OK;
}

// Rows are bucketed by length; each bucket has its own kernel shape: several rows per wavefront
// up to 32 elements, one wavefront per row for short rows, one workgroup per row above.
template <typename KeyT, int CODEC, bool HAS_IDX>
inline int sort_rows_in_lds(const SortRequest& r)
{
  if (r.row_stride != 0 && (r.seg <= 4096 || sizeof(KeyT) < 4)) {
    return CPN_ERR_UNSUPPORTED;  // only the one-workgroup-per-row kernel of 4- and 8-byte keys takes strided rows
  }
  if (r.volume / r.seg * r.pieces >= (1ull << 31)) {
    return CPN_ERR_UNSUPPORTED;
  }
  if constexpr (sizeof(KeyT) <= 8 && (CODEC == CODEC_UNSIGNED || CODEC == CODEC_SIGNED || CODEC == CODEC_FLOAT)) {
    // (Rows just past 32 and 64 keys used to be sorted by counting, for every key, the keys of its row that come
    // before it, because the network ran in the next power of two of slots: 2^26 float32 keys in rows of 33 with
    // positions 0.33 ms counted, 0.15 in the network since a row takes 4 lanes of 10 elements.)
    // rows of 2 ... 128 keys and more (bitonic_row_limit): a sorting network on eight to fourteen elements per lane
    if (r.seg >= 2 && r.seg <= bitonic_row_limit(sizeof(KeyT), HAS_IDX, CODEC == CODEC_FLOAT) && r.seg <= wave_row_limit() &&
        bitonic_rows_enabled()) {
      if constexpr (!HAS_IDX && sizeof(KeyT) == 8) {
        // full rows of a power of two of 8-byte keys, values only: sixteen elements per lane
        if (r.seg == 32) {
          return launch_bitonic_rows<KeyT, CODEC, HAS_IDX, 2, 16>(r);
        } else if (r.seg == 64) {
          return launch_bitonic_rows<KeyT, CODEC, HAS_IDX, 4, 16>(r);
        } else if (r.seg == 128) {
          return launch_bitonic_rows<KeyT, CODEC, HAS_IDX, 8, 16>(r);
        } else if (r.seg == 256) {
          return launch_bitonic_rows<KeyT, CODEC, HAS_IDX, 16, 16>(r);
        }
      }
      if (r.seg <= 8) {
        return launch_bitonic_rows<KeyT, CODEC, HAS_IDX, 1, 8>(r);
      } else if (r.seg <= 16) {
        return launch_bitonic_rows<KeyT, CODEC, HAS_IDX, 2, 8>(r);
      } else if (r.seg <= 32) {
        return launch_bitonic_lanes<KeyT, CODEC, HAS_IDX, 4>(r);
      } else if (r.seg <= 64) {
        return launch_bitonic_lanes<KeyT, CODEC, HAS_IDX, 8>(r);
      } else if (r.seg <= 128) {
        return launch_bitonic_lanes<KeyT, CODEC, HAS_IDX, 16>(r);
      } else if (r.seg <= 256) {
        return launch_bitonic_lanes<KeyT, CODEC, HAS_IDX, 32>(r);
      }
      if constexpr (sizeof(KeyT) == 8 && CODEC == CODEC_FLOAT && !HAS_IDX) {
        // 257 ... 384 float64 keys, values only (compared as numbers): 32 lanes of 10 or 12
        if (r.seg <= 320) {
          return launch_bitonic_rows<KeyT, CODEC, HAS_IDX, 32, 10>(r);
        }
        return launch_bitonic_rows<KeyT, CODEC, HAS_IDX, 32, 12>(r);
      }
      if constexpr (sizeof(KeyT) == 2 || sizeof(KeyT) == 4) {
        // a row per wavefront: 8 ... 16 elements per lane
        if (r.seg <= 512) {
          return launch_bitonic_lanes<KeyT, CODEC, HAS_IDX, 64>(r);
        }
        const uint64_t e = (r.seg + WAVE - 1) / WAVE;
        if (e <= 10) {
          return launch_bitonic_rows<KeyT, CODEC, HAS_IDX, 64, 10>(r);
        } else if (e <= 12) {
          return launch_bitonic_rows<KeyT, CODEC, HAS_IDX, 64, 12>(r);
        } else if (e <= 14) {
          return launch_bitonic_rows<KeyT, CODEC, HAS_IDX, 64, 14>(r);
        }
        return launch_bitonic_rows<KeyT, CODEC, HAS_IDX, 64, 16>(r);
      }
    }
  }
  if (r.seg <= 32 && r.seg <= wave_row_limit()) {
    if (r.seg <= 1) {
      return launch_tiny_rows<KeyT, CODEC, HAS_IDX, 1>(r);
    } else if (r.seg <= 2) {
      return launch_tiny_rows<KeyT, CODEC, HAS_IDX, 2>(r);
    } else if (r.seg <= 4) {
      return launch_tiny_rows<KeyT, CODEC, HAS_IDX, 4>(r);
    } else if (r.seg <= 8) {
      return launch_tiny_rows<KeyT, CODEC, HAS_IDX, 8>(r);
    } else if (r.seg <= 16) {
      return launch_tiny_rows<KeyT, CODEC, HAS_IDX, 16>(r);
    } else {
      return launch_tiny_rows<KeyT, CODEC, HAS_IDX, 32>(r);
    }
  }
  if ((sizeof(KeyT) == 4 || sizeof(KeyT) == 8) && r.seg > 256 && r.seg <= 512 && CODEC != CODEC_COMPLEX) {
    // real keys of 4 and 8 bytes: the workgroup kernel in a one-wave shape, eight keys per lane, split into
    // value ranges, ahead of the one-wave ranking kernel: 2^26 float64 keys in rows of 512 0.32 -> 0.23 ms,
    // of 257 0.57 -> 0.40; float32 rows of 512 0.24 -> 0.21, argsort 0.31 -> 0.29
    return launch_lds_rows<KeyT, CODEC, HAS_IDX, 64, 8>(r);
  }
  if ((sizeof(KeyT) == 4 || sizeof(KeyT) == 8) && r.seg > 128 && r.seg <= 256 && CODEC != CODEC_COMPLEX) {
    // (the same with four keys per lane: float32 rows of 256 0.27 -> 0.22 ms, float64 rows of 256 0.35 -> 0.29,
    // of 129 0.69 -> 0.52, with positions 0.72 -> 0.45)
    return launch_lds_rows<KeyT, CODEC, HAS_IDX, 64, 4>(r);
  }
  // The one-wave ranking kernel: keys of 1 and 2 bytes up to 1024, the others up to 512 (keys of 8 bytes
  // and more hold too many registers per lane at 16 items, and for 4-byte keys the workgroup kernel with
  // its split into value ranges is the faster one: 2^26 float32 keys in rows of 513 0.63 -> 0.38 ms, of
  // 1024 0.34 -> 0.23, argsort of rows of 1024 0.44 -> 0.31; rows of 1024 float16 keys 0.17 against
  // 0.20 ms, of single bytes 0.067 against 0.081).  Real keys of 4 and 8 bytes have left above.
  if (r.seg <= wave_row_limit() && (sizeof(KeyT) < 4 || r.seg <= 512)) {
    if (r.seg <= 64) {
      return launch_wave_rows<KeyT, CODEC, HAS_IDX, 1>(r);
    } else if (r.seg <= 128) {
      return launch_wave_rows<KeyT, CODEC, HAS_IDX, 2>(r);
    } else if (r.seg <= 256) {
      return launch_wave_rows<KeyT, CODEC, HAS_IDX, 4>(r);
    } else if (r.seg <= 512) {
      return launch_wave_rows<KeyT, CODEC, HAS_IDX, 8>(r);
    } else {
      return launch_wave_rows<KeyT, CODEC, HAS_IDX, 16>(r);
    }
  }
  if constexpr (sizeof(KeyT) == 2 && !HAS_IDX && CODEC != CODEC_COMPLEX) {
    // values only, 2-byte keys: long rows are counted instead of ranked
    if (r.seg >= count16_min_row() && r.seg >= 64) {
      return launch_count16_rows<CODEC>(r);
    }
  }
  if (r.seg <= 64) {
    return launch_lds_rows<KeyT, CODEC, HAS_IDX, 64, 1>(r);
  } else if (r.seg <= 256) {
    return launch_lds_rows<KeyT, CODEC, HAS_IDX, 64, 4>(r);
  } else if ((sizeof(KeyT) == 4 || sizeof(KeyT) == 8) && r.seg <= 768) {
    // one wavefront per row, twelve keys per lane, split into value ranges: 2^26 float32 keys in rows of
    // 513 0.39 -> 0.25 ms, of 768 0.29 -> 0.23; float64 rows of 513 0.43 -> 0.34
    return launch_lds_rows<KeyT, CODEC, HAS_IDX, 64, 12>(r);
  } else if (r.seg <= 1024) {
    return launch_lds_rows<KeyT, CODEC, HAS_IDX, 128, 8>(r);
  } else if ((sizeof(KeyT) == 4 || sizeof(KeyT) == 8) && r.seg <= 1536) {
    // twelve keys per thread: a step between the shapes of 1024 and 2048 keys for the keys that are split
    // into value ranges (2^26 float32 keys in rows of 1025 0.40 -> 0.31 ms, of 1536 0.30 -> 0.25)
    return launch_lds_rows<KeyT, CODEC, HAS_IDX, 128, 12>(r);
  } else if (r.seg <= 2048) {
    return launch_lds_rows<KeyT, CODEC, HAS_IDX, 256, 8>(r);
  }
  if constexpr (sizeof(KeyT) == 16) {
    return launch_lds_rows<KeyT, CODEC, HAS_IDX, 1024, 4>(r);  // lds_row_capacity(16) == 4096
  } else {
    if constexpr (sizeof(KeyT) == 4 || sizeof(KeyT) == 8) {
      if (r.seg <= 3072) {
        // (the same between 2048 and 4096: rows of 2049 float32 keys 0.42 -> 0.32 ms, of 3072 0.32 -> 0.25;
        // argsort of float64 rows of 2049 0.65 -> 0.52)
        return launch_lds_rows<KeyT, CODEC, HAS_IDX, 256, 12>(r);
      }
    }
    if (r.seg <= 4096) {
      // eight keys per thread when a thread also carries positions (10-25 % faster than sixteen) and
      // for keys of 4 and 8 bytes, whose rows are split into value ranges (twice the waves per CU:
      // 2^26 float32 keys in rows of 4096 0.33 -> 0.27 ms, of 2049 0.57 -> 0.42); sixteen for plain
      // sorts of 1- and 2-byte keys
      if constexpr (HAS_IDX || sizeof(KeyT) >= 4) {
        return launch_lds_rows<KeyT, CODEC, HAS_IDX, 512, 8>(r);
      } else {
        return launch_lds_rows<KeyT, CODEC, HAS_IDX, 256, 16>(r);
      }
    }
    if constexpr (sizeof(KeyT) == 8) {
      // 512 threads with 12 or 16 keys each leave room for two workgroups on a CU (48 or 64 KiB of keys
      // and a small table of bins), which 1024 threads x 8 do not: 2^26 float64 keys in rows of 4097
      // 0.89 -> 0.47 ms, of 6144 0.70 -> 0.36
      if (r.seg <= 6144) {
        return launch_lds_rows<KeyT, CODEC, HAS_IDX, 512, 12>(r);
      }
      if (r.seg <= 8192) {
        if constexpr (!HAS_IDX) {
          return launch_lds_rows<KeyT, CODEC, HAS_IDX, 512, 16>(r);
        } else {
          return launch_lds_rows<KeyT, CODEC, HAS_IDX, 1024, 8>(r);  // (the staged positions take the room)
        }
      }
      // the longest rows that fit the LDS of a CU: lds_row_capacity(8, HAS_IDX)
      return launch_lds_rows<KeyT, CODEC, HAS_IDX, 1024, (HAS_IDX ? 14 : 16)>(r);
    } else {
      if (r.seg <= 8192) {
        // sixteen waves of eight keys hide the ranking latency better than eight waves of sixteen
        // (4-12 % on 2- and 4-byte keys); one-pass sorts of single bytes prefer fewer barriers
        if constexpr (sizeof(KeyT) == 1) {
          return launch_lds_rows<KeyT, CODEC, HAS_IDX, 512, 16>(r);
        } else if constexpr (sizeof(KeyT) == 2) {
          // 2-byte keys: two passes in 512-thread shapes, two workgroups per CU; for plain sorts ahead of the
          // counting kernel up to here (2^26 float16 keys in rows of 4097 0.39 -> 0.27 ms, of 8192 0.20 -> 0.18;
          // with positions, against 1024 threads x 8 keys: rows of 6144 0.40 -> 0.36, of 8192 0.35 -> 0.32)
          if (r.seg <= 6144) {
            return launch_lds_rows<KeyT, CODEC, HAS_IDX, 512, 12>(r);
          }
          return launch_lds_rows<KeyT, CODEC, HAS_IDX, 512, 16>(r);
        } else if constexpr (sizeof(KeyT) == 4) {
          // (split into value ranges: two workgroups of 512 threads on a CU, as for 8-byte keys above)
          if (r.seg <= 6144) {
            return launch_lds_rows<KeyT, CODEC, HAS_IDX, 512, 12>(r);
          }
          return launch_lds_rows<KeyT, CODEC, HAS_IDX, 512, 16>(r);
        } else {
          return launch_lds_rows<KeyT, CODEC, HAS_IDX, 1024, 8>(r);
        }
      }
      if constexpr (sizeof(KeyT) == 4 && !HAS_IDX) {
        if (r.seg <= 12288) {
          return launch_lds_rows<KeyT, CODEC, HAS_IDX, 512, 24>(r);  // two workgroups per CU, as above
        }
      }
      // (2-byte keys, values only, come here when the counting kernel is switched off or starts later.  A
      // 512 x 32 shape for them, two workgroups per CU and rows dealt in equal shares, measured 0.35 ms for
      // 2^26 float16 keys in rows of 8193 and 0.27 in rows of 16 384 against the counting kernel's 0.38 and
      // 0.19: not kept)
      return launch_lds_rows<KeyT, CODEC, HAS_IDX, 1024, 16>(r);  // up to 16 384 keys
    }
  }
}

// ---- global onesweep path --------------------------------------------------------------
template <typename KeyT, int CODEC, bool BIG, bool HAS_IDX>
inline int sort_global(const SortRequest& r, const GlobalLayout& L)
{
  using OffT           = typename RowWidth<BIG>::off_t;
  constexpr int KB     = sizeof(KeyT);
  constexpr int BLOCK  = global_block(KB);
  constexpr int ITEMS  = global_items(KB, BIG);
  constexpr int PASSES = KeyTraits<CODEC, KeyT>::PASSES;
  unsigned char* ws    = static_cast<unsigned char*>(r.temp);
  const bool in_place  = (r.values_out == r.values_in);
  const bool want_vals = (r.values_out != nullptr);

  int rc = launch_zero_fill(ws, L.zero_bytes, r.stream);
  if (rc != CPN_OK) {
    return rc;
  }
  uint32_t* status  = reinterpret_cast<uint32_t*>(ws);
  uint32_t* tickets = reinterpret_cast<uint32_t*>(ws + HEADER_TICKETS);
  uint32_t* varying = reinterpret_cast<uint32_t*>(ws + HEADER_VARYING);
  SortPlan* plan    = reinterpret_cast<SortPlan*>(ws + HEADER_PLAN);
  constexpr bool VIRT_OK = !BIG && KB == 8 && KeyTraits<CODEC, KeyT>::PASSES == KB;
  VirtPlan* vplan   = L.virt ? reinterpret_cast<VirtPlan*>(ws + L.off_virt) : nullptr;
  DistinctTable* dtable = L.virt ? reinterpret_cast<DistinctTable*>(ws + L.off_virt + VIRT_PLAN_BYTES) : nullptr;
  OffT* hist        = reinterpret_cast<OffT*>(ws + L.off_hist);
  static_assert(PASSES <= MAX_PASSES, "plan table too small");
  PlanRequest rq{};
  rq.passes       = PASSES;
  rq.want_values  = want_vals ? 1u : 0u;
  rq.want_indices = HAS_IDX ? 1u : 0u;
  rq.in_place     = in_place ? 1u : 0u;
  rq.free_rank    = (!HAS_IDX && (CODEC == CODEC_UNSIGNED || CODEC == CODEC_SIGNED || CODEC == CODEC_FLOAT)) ? 1u : 0u;
  rq.specials     = (CODEC == CODEC_FLOAT) ? reinterpret_cast<const uint32_t*>(ws + HEADER_SPECIALS) : nullptr;

  // histogram sweep: about 2048 blocks in total, at least one per row
  {
    uint64_t bpr = 2048 / L.rows;
    if (bpr < 1) {
      bpr = 1;
    }
    const uint64_t min_chunk = 16384;
    const uint64_t max_bpr   = (r.seg + min_chunk - 1) / min_chunk;
    if (bpr > max_bpr) {
      bpr = max_bpr;
    }
    uint64_t chunk = (r.seg + bpr - 1) / bpr;
    chunk          = align_up(chunk, 4096);
    bpr            = (r.seg + chunk - 1) / chunk;
    const uint64_t grid = bpr * L.rows;
    if (grid >= (1ull << 31)) {
      return CPN_ERR_UNSUPPORTED;
    }
    if constexpr (VIRT_OK) {
      if (L.virt) {
        // At most 256 different keys in the row?  A sample decides whether it is worth finding out;
        // if so a sweep collects the keys and a plan kernel sets up the one pass on their ranks,
        // and the histogram sweep and the other plan kernels below then exit at once.
        {
          ProfileScope prof("distinct_sample", r.stream);
          hipLaunchKernelGGL((distinct_sample_kernel<KeyT, CODEC>), dim3(1), dim3(RADIX), 0, r.stream,
                             static_cast<const KeyT*>(r.values_in), r.seg, dtable);
        }
        CPN_HIP_TRY(hipGetLastError());
        {
          const uint64_t dchunk = 65536;
          const uint64_t dgrid  = (r.seg + dchunk - 1) / dchunk;
          ProfileScope prof("distinct_sweep", r.stream);
          hipLaunchKernelGGL((distinct_sweep_kernel<KeyT, CODEC>), dim3(static_cast<uint32_t>(dgrid)), dim3(DSWEEP_BLOCK),
                             0, r.stream, static_cast<const KeyT*>(r.values_in), r.seg, dchunk, dtable);
        }
        CPN_HIP_TRY(hipGetLastError());
        {
          ProfileScope prof("distinct_plan", r.stream);
          hipLaunchKernelGGL((distinct_plan_kernel<OffT>), dim3(1), dim3(RADIX), 0, r.stream, hist, varying, vplan,
                             dtable, r.seg, static_cast<uint32_t>(PASSES));
        }
        CPN_HIP_TRY(hipGetLastError());
      }
    }
    {
      ProfileScope prof("histogram", r.stream);
      constexpr bool SPECIALS = (CODEC == CODEC_FLOAT) && !HAS_IDX;  // who may rank its first pass freely
      hipLaunchKernelGGL((histogram_kernel<KeyT, CODEC, OffT, SPECIALS>), dim3(static_cast<uint32_t>(grid)),
                         dim3(HIST_BLOCK), 0, r.stream, static_cast<const KeyT*>(r.values_in), hist, r.seg,
                         static_cast<uint32_t>(bpr), chunk, static_cast<const VirtPlan*>(vplan),
                         reinterpret_cast<uint32_t*>(ws + HEADER_SPECIALS));
    }
    CPN_HIP_TRY(hipGetLastError());
    {
      ProfileScope prof("histogram_scan", r.stream);
      const uint64_t n_hist = L.rows * PASSES;
      uint64_t sgrid        = (n_hist + SCAN_BLOCK / WAVE - 1) / (SCAN_BLOCK / WAVE);
      // Every workgroup ends with one atomic on the same word (the last one makes the plan), and those
      // queue: 4092 histograms on 1023 workgroups took 0.087 ms, on 64 workgroups 0.021 ms.
      const uint64_t sgrid_cap = n_hist / 64 < 64 ? 64 : (n_hist / 64 > 1024 ? 1024 : n_hist / 64);
      if (sgrid > sgrid_cap) {
        sgrid = sgrid_cap;
      }
      hipLaunchKernelGGL((histogram_scan_kernel<OffT>), dim3(static_cast<uint32_t>(sgrid)), dim3(SCAN_BLOCK), 0,
                         r.stream, hist, varying, r.seg, static_cast<uint32_t>(PASSES), n_hist,
                         static_cast<const VirtPlan*>(vplan), 0u,
                         L.virt ? nullptr : reinterpret_cast<uint32_t*>(ws + HEADER_SCAN_DONE), plan, rq);
    }
    CPN_HIP_TRY(hipGetLastError());
    if constexpr (VIRT_OK) {
      if (L.virt) {
        // may replace the byte passes by fewer passes on virtual digits (decided on the device)
        {
          ProfileScope prof("virtual_plan", r.stream);
          hipLaunchKernelGGL((vplan_kernel<OffT>), dim3(1), dim3(RADIX), 0, r.stream, hist, varying, vplan, r.seg,
                             static_cast<uint32_t>(PASSES));
        }
        CPN_HIP_TRY(hipGetLastError());
        {
          const uint64_t vchunk = 65536;
          const uint64_t vgrid  = (r.seg + vchunk - 1) / vchunk;
          ProfileScope prof("virtual_histogram", r.stream);
          hipLaunchKernelGGL((vhist_kernel<KeyT, CODEC, OffT>), dim3(static_cast<uint32_t>(vgrid)), dim3(VHIST_BLOCK), 0,
                             r.stream, static_cast<const KeyT*>(r.values_in), hist, vplan, r.seg, vchunk);
        }
        CPN_HIP_TRY(hipGetLastError());
        {
          ProfileScope prof("virtual_scan", r.stream);
          hipLaunchKernelGGL((histogram_scan_kernel<OffT>), dim3((PASSES + SCAN_BLOCK / WAVE - 1) / (SCAN_BLOCK / WAVE)),
                             dim3(SCAN_BLOCK), 0, r.stream, hist, varying, r.seg, static_cast<uint32_t>(PASSES),
                             static_cast<uint64_t>(PASSES), vplan, 1u, static_cast<uint32_t*>(nullptr), plan, rq);
        }
        CPN_HIP_TRY(hipGetLastError());
      }
    }
    if (L.virt) {  // otherwise the scan kernel has made the plan
      ProfileScope prof("plan", r.stream);
      hipLaunchKernelGGL(plan_kernel, dim3(1), dim3(WAVE), 0, r.stream, varying, plan, rq);
      CPN_HIP_TRY(hipGetLastError());
    }
  }

  // The buffers a pass may read or write; which ones it uses is in the device-side plan.
  void* key1 = L.off_key1 ? ws + L.off_key1 : nullptr;
  void* key2 = L.off_key2 ? ws + L.off_key2 : nullptr;
  void* idx1 = L.off_idx ? ws + L.off_idx : nullptr;

  // Index-only sorts never return the keys: the first running pass stores their
  // order-preserving unsigned image and every pass extracts digits with the identity codec.
  constexpr bool CAN_ORDER_KEYS = HAS_IDX && (CODEC == CODEC_SIGNED || CODEC == CODEC_FLOAT) && PASSES >= 2;
  const bool ordered_keys       = CAN_ORDER_KEYS && !want_vals;

  // Index-only requests that may run on the ranks of the row's different keys: that one pass (the
  // device-side plan says whether it is to run) in a shape of its own, 512 threads x 32 keys with one
  // byte per key in LDS, two workgroups per CU; the launch of pass 0 below then finds it done.
  // Measured on 2^27 int64 keys drawn from 16 values: the pass 0.70 ms in the 1024-thread shape,
  // whose one workgroup per CU runs its phases one after the other.
  constexpr bool DISTINCT_SPECIAL = VIRT_OK && HAS_IDX && global_block(KB) * global_items(KB, BIG) == 512 * 32;
  const bool distinct_special     = DISTINCT_SPECIAL && L.virt && !want_vals;
  auto pass_args = [&](int p) {
    SweepArgs<BIG> a{};
    a.key_buf[KEY_IN]    = r.values_in;
    a.key_buf[KEY_OUT]   = r.values_out;
    a.key_buf[KEY_T1]    = key1;
    a.key_buf[KEY_T2]    = key2;
    a.idx_buf[0]         = nullptr;
    a.idx_buf[IDX_FINAL] = r.indices_out;
    a.idx_buf[IDX_T1]    = idx1;
    a.idx_buf[IDX_ALIAS] = r.indices_out;
    a.plan               = plan;
    a.ticket             = tickets + p;
    a.xcd_tickets        = reinterpret_cast<uint32_t*>(ws + HEADER_XCD_TICKETS) + p * XCD_COUNT;
    a.hist_excl          = hist + p * RADIX;
    a.desc               = reinterpret_cast<OffT*>(ws + L.off_desc + L.desc_bytes_per_pass * p);
    a.status             = status;
    a.seg                = r.seg;
    a.hist_row_stride    = static_cast<uint64_t>(PASSES) * RADIX;
    a.index_offset       = r.index_offset;
    a.tiles_per_row      = L.tiles_per_row;
    a.num_tiles          = static_cast<uint32_t>(L.num_tiles);
    a.pass               = p;
    a.spin_limit         = lookback_spin_limit();
    a.single_ticket      = (r.single_ticket || tile_order_single()) ? 1u : 0u;
    a.vplan              = vplan;
    a.dtable             = dtable;
    a.distinct_pass_done = distinct_special ? 1u : 0u;
    return a;
  };
  if constexpr (DISTINCT_SPECIAL) {
    if (distinct_special) {
      const SweepArgs<BIG> a = pass_args(0);
      ProfileScope prof("onesweep_distinct", r.stream);
      hipLaunchKernelGGL((onesweep_kernel<KeyT, CODEC, false, BIG, HAS_IDX, 512, 32, true, true>),
                         dim3(static_cast<uint32_t>(L.num_tiles)), dim3(512), 0, r.stream, a);
      CPN_HIP_TRY(hipGetLastError());
    }
  }
  for (int p = 0; p < PASSES; ++p) {
    const SweepArgs<BIG> a = pass_args(p);
    {
      ProfileScope prof("onesweep", r.stream);
      const dim3 grid(static_cast<uint32_t>(L.num_tiles));
      // requests that may run on virtual digits get the kernel that can do both (the device-side
      // plan decides); everything else the plain one
      bool launched = false;
      if constexpr (VIRT_OK) {
        if (L.virt) {
          if constexpr (CAN_ORDER_KEYS) {
            if (ordered_keys) {
              hipLaunchKernelGGL((onesweep_kernel<KeyT, CODEC, true, BIG, HAS_IDX, BLOCK, ITEMS, true>), grid,
                                 dim3(BLOCK), 0, r.stream, a);
              launched = true;
            }
          }
          if (!launched) {
            hipLaunchKernelGGL((onesweep_kernel<KeyT, CODEC, false, BIG, HAS_IDX, BLOCK, ITEMS, true>), grid,
                               dim3(BLOCK), 0, r.stream, a);
            launched = true;
          }
        }
      }
      if constexpr (CAN_ORDER_KEYS) {
        if (!launched && ordered_keys) {
          hipLaunchKernelGGL((onesweep_kernel<KeyT, CODEC, true, BIG, HAS_IDX, BLOCK, ITEMS>), grid, dim3(BLOCK), 0,
                             r.stream, a);
          launched = true;
        }
      }
      if (!launched) {
        hipLaunchKernelGGL((onesweep_kernel<KeyT, CODEC, false, BIG, HAS_IDX, BLOCK, ITEMS>), grid, dim3(BLOCK), 0,
                           r.stream, a);
      }
    }
    CPN_HIP_TRY(hipGetLastError());
  }
  {
    uint64_t blocks = (r.volume + 1023) / 1024;
    if (blocks > 8192) {
      blocks = 8192;
    }
    ProfileScope prof("finalize", r.stream);
    hipLaunchKernelGGL((finalize_kernel<KeyT>), dim3(static_cast<uint32_t>(blocks)), dim3(256), 0, r.stream, plan,
                       static_cast<const KeyT*>(r.values_in), static_cast<KeyT*>(r.values_out),
                       static_cast<const KeyT*>(key1), r.indices_out, r.volume, r.seg, r.index_offset, rq);
  }
  CPN_HIP_TRY(hipGetLastError());
  return CPN_OK;
}

template <typename KeyT, int CODEC>
int sort_typed(const SortRequest& r)
{
  constexpr int KB     = sizeof(KeyT);
  constexpr int PASSES = KeyTraits<CODEC, KeyT>::PASSES;
  const bool has_idx   = (r.indices_out != nullptr);
  const bool in_place  = (r.values_out == r.values_in);
  const uint64_t need  = workspace_bytes(KB, PASSES, r.volume, r.seg, r.values_out != nullptr, has_idx, in_place);
  if (need == 0) {
    return CPN_ERR_UNSUPPORTED;
  }
  if (r.temp == nullptr || r.temp_bytes < need || (reinterpret_cast<uintptr_t>(r.temp) % WORKSPACE_ALIGN) != 0) {
    return CPN_ERR_TEMP;
  }
  if (r.seg <= lds_row_limit(KB, has_idx)) {
    // one launch: the row kernels clear the status word of the workspace themselves.  (More rows than a
    // grid can have blocks, e.g. a (2^31, 1) array: one launch per 2^30 rows.)
    constexpr uint64_t ROWS_PER_LAUNCH = 1ull << 30;
    const uint64_t rows                = r.volume / r.seg;
    for (uint64_t first = 0; first < rows; first += ROWS_PER_LAUNCH) {
      const uint64_t count = rows - first < ROWS_PER_LAUNCH ? rows - first : ROWS_PER_LAUNCH;
      SortRequest c        = r;
      c.volume             = count * r.seg;
      c.values_in          = static_cast<const KeyT*>(r.values_in) + first * r.seg;
      c.values_out         = r.values_out != nullptr ? static_cast<KeyT*>(r.values_out) + first * r.seg : nullptr;
      c.indices_out        = r.indices_out != nullptr ? r.indices_out + first * r.seg : nullptr;
      const int rc         = has_idx ? sort_rows_in_lds<KeyT, CODEC, true>(c) : sort_rows_in_lds<KeyT, CODEC, false>(c);
      if (rc != CPN_OK) {
        return rc;
      }
    }
    return CPN_OK;
  }
  if constexpr ((KB == 4 || KB == 8) && KeyTraits<CODEC, KeyT>::NWORDS == 1) {
    if (const int levels = merged_row_levels(KB, PASSES, r.volume, r.seg, has_idx); levels != 0) {
      return has_idx ? sort_rows_merged<KeyT, CODEC, true>(r, levels) : sort_rows_merged<KeyT, CODEC, false>(r, levels);
    }
  }
  const GlobalLayout L = global_layout(KB, PASSES, r.volume, r.seg, r.values_out != nullptr, has_idx, in_place);
  if (L.big) {
    return has_idx ? sort_global<KeyT, CODEC, true, true>(r, L) : sort_global<KeyT, CODEC, true, false>(r, L);
  }
  return has_idx ? sort_global<KeyT, CODEC, false, true>(r, L) : sort_global<KeyT, CODEC, false, false>(r, L);
}

// One translation unit per key width instantiates these (keeps hipcc runs parallel).
int sort_keys8(int codec, const SortRequest& r);
int sort_keys16(int codec, const SortRequest& r);
int sort_keys32(int codec, const SortRequest& r);
int sort_keys64(int codec, const SortRequest& r);
int sort_keys128(int codec, const SortRequest& r);

}  // namespace cpn
