// Per-row sort in LDS: one workgroup owns one row (up to BLOCK*ITEMS elements), keeps the
// keys in registers and runs a stable 8-bit LSD radix sort whose exchange step goes through
// LDS.  One read and one write of HBM per element, whatever the key width.
//
// Replaces, for rows that fit, cub::DeviceSegmentedRadixSort
// (src/cupynumeric/sort/cub_sort.cuh:81-105,153-182) and the (segment id, value) tuple
// merge sort used for rows of at most 400 elements (src/cupynumeric/sort/thrust_sort.cuh:68-122).
//
// Digits on which every key of the row agrees are found up front with one AND/OR
// reduction and their passes are skipped (the pass would be the identity permutation).
//
// All loads of a row are issued before the first use, unconditionally, from offsets clamped into
// the row: under the branch that also encodes a key the compiler waits for each load before it
// issues the next, and under per-round uniform branches it copies the whole key array at every
// join and spills.
//
// Wide keys: a row of n keys is almost always put in order by its leading 2*log2(n) or so
// varying bits.  When more passes than that are due, the kernel first runs only the passes of
// the most significant varying digits, then checks that every neighbouring pair of the result
// is in order on the whole key.  If so the row is sorted (stably: ties on the leading digits
// whose remaining digits also tie kept their input order).  If a few pairs are not, rounds of
// odd-even transposition between neighbours repair them; if that does not finish within
// FIXUP_ROUNDS, all passes are run, from the state reached, which is still a stable sort of
// the input.
//
// Values-only sorts of rows whose keys that tie are the same bits (integers; floats without NaN and
// -0.0): no order among equal keys shows, so the row need not go through stable passes at all.  It
// is first split into 8192 ranges (bins) of equal width between its smallest and its largest key
// (4096 for tiles of more than 64 KiB, whose bins share the memory of the digit counters), one LDS
// atomic per key, which leaves a handful of keys per bin on evenly or normally distributed data; a
// second atomic puts every key into its bin and tells the key where it went; every key then finds
// its place inside its bin by counting the keys of the bin that come before it.  A row that
// crowds more than BUCKET_LIMIT keys into one bin (few different keys, tight clusters) goes
// through the radix passes instead.  Used by every shape of at least four keys per thread, for real
// keys of 4 or 8 bytes (the one-wave ranking kernel, wave_row_sort.h, has the same path for 4-byte keys); the number of bins is bucket_bins_log2.  Sorts that carry positions take
// it as well: the position a key came from is staged beside the key and breaks the ties inside a
// bin, which makes the result the stable order.
//
// Floating-point rows without NaN and without -0.0 (found during the same reduction): on such
// a row the ordered image of a key is a bijection of its bits, so the keys are replaced by
// their images once, the passes take plain bytes of them, and the images are mapped back
// before the store.  Rows with a NaN or a -0.0 keep the raw bits and apply the codec per pass
// (so do all float16 rows and the rows sorted by 1024 threads).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <limits>
#include <type_traits>

#include "radix_common.h"
#include "wave_row_sort.h"  // wave_all_and / wave_all_or, FIXUP_ROUNDS

namespace cpn {

// Bins of the split above: 8192 where they fit beside the row (and the staged positions of an
// argsort), 4096 (which share the 16 KiB of the digit counters) where that keeps two workgroups on a
// CU or where nothing more is left of the CU's 160 KiB.
__host__ __device__ constexpr int bucket_bins_log2(int tile, int key_bytes, bool has_idx, int block)
{
  const int row_bytes = tile * key_bytes + (has_idx ? tile * 2 : 0);
  constexpr int KIB = 1024;
  if (tile <= 256) {
    return 8;  // one bin per key
  }
  if (tile <= 4096) {
    // One bin per key; two for plain sorts of 4-byte keys.  More bins shorten the walks and cost LDS,
    // i.e. workgroups per CU, which weighs more.  Measured on 2^26 keys, two / one / half a bin per key:
    // rows of 1024 float64 0.28 / 0.26 / 0.26 ms (four per key: 0.43), 2048 float64 0.34 / 0.28 / 0.30,
    // 4096 float64 0.38 / 0.32 / 0.33, 4096 float32 with positions 0.39 / 0.34 / 0.41, and plain
    // 4096 float32 0.275 / 0.281 / 0.327, 2048 float32 0.259 / 0.266 / 0.302.
    // (The shapes of 12 keys per thread, tiles of 1536 and 3072 keys, keep the table of the next smaller
    // power of two: 1.33 bins per key; with 2.67 rows of 3072 float32 keys took 0.37 ms instead of 0.25.)
    // (The one-wave shape of 768 keys: 512 bins for plain sorts, 2^26 float32 keys in rows of 513 0.25 ms
    // against 0.28 with 1024 bins; 1024 with positions, 0.305 against 0.32 ms for rows of 768.)
    return (tile <= 1024 ? 10 : (tile <= 2048 ? 11 : 12)) + ((key_bytes == 4 && !has_idx && tile % 3 != 0) ? 1 : 0) -
           ((tile <= 768 && !has_idx) ? 1 : 0);
  }
  if (row_bytes + 32 * KIB <= 78 * KIB) {
    return 13;  // two workgroups per CU either way
  }
  if (row_bytes + 16 * KIB <= 78 * KIB) {
    return 12;  // two workgroups per CU only with the smaller table
  }
  if (block <= 512 && row_bytes + 8 * KIB <= 78 * KIB) {
    // 8192 eight-byte keys on 512 threads: a quarter of a bin per key, and two workgroups per CU
    // (1024 threads with more than 64 registers each have a CU to themselves anyway)
    return 11;
  }
  return row_bytes + 32 * KIB <= 158 * KIB ? 13 : 12;
}
// Most keys a bin may hold for the split to be used (each key of a bin is compared with all others).
constexpr uint32_t BUCKET_LIMIT = 24;
// (four keys per bin on average instead of one or two, in the shape with 4096 bins for up to 16 384 keys)
#ifndef CPN_BUCKET_LIMIT_WIDE
#define CPN_BUCKET_LIMIT_WIDE 48
#endif
constexpr uint32_t BUCKET_LIMIT_WIDE = CPN_BUCKET_LIMIT_WIDE;
// Keys past the end of a bin that the walk over the bins may read (and not count).
constexpr int BUCKET_PAD = 64;

// The arithmetic type of a real key of 4 or 8 bytes.
template <int CODEC, int BYTES>
struct NativeKey {
  using type = uint32_t;
};
template <> struct NativeKey<CODEC_UNSIGNED, 8> { using type = uint64_t; };
template <> struct NativeKey<CODEC_SIGNED, 4> { using type = int32_t; };
template <> struct NativeKey<CODEC_SIGNED, 8> { using type = int64_t; };
template <> struct NativeKey<CODEC_FLOAT, 4> { using type = float; };
template <> struct NativeKey<CODEC_FLOAT, 8> { using type = double; };

// Waves per SIMD the compiler has to leave room for.  1024 threads with 8 keys of up to 4 bytes each stay below 64
// vector registers and 80 KiB of LDS so that two workgroups share a CU; that also takes at most
// 100 scalar registers per wave, which the compiler exceeds unless it is told (it then keeps a
// few uniform values in vector registers instead).
__host__ __device__ constexpr int lds_row_waves_per_simd(int block, int items, int key_bytes)
{
  return (block == 1024 && items <= 8 && key_bytes <= 4) ? 8 : 1;
}

template <typename KeyT, int CODEC, bool HAS_IDX, int BLOCK, int ITEMS>
__global__ __launch_bounds__(BLOCK) __attribute__((amdgpu_waves_per_eu(lds_row_waves_per_simd(BLOCK, ITEMS, sizeof(KeyT)))))
void lds_row_sort_kernel(const KeyT* keys_in,
                                                              KeyT* keys_out,
                                                              int64_t* idx_out,
                                                              uint32_t piece_len,
                                                              uint64_t row_stride,
                                                              uint32_t pieces,
                                                              uint32_t last_piece_len,
                                                              int64_t index_offset,
                                                              uint32_t* status)
{
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    *status = 0;  // the workspace's status word: a per-row sort cannot fail on the device
  }
  constexpr int WAVES  = BLOCK / WAVE;
  constexpr int TILE   = BLOCK * ITEMS;
  constexpr int WTILE  = ITEMS * WAVE;
  using KT             = KeyTraits<CODEC, KeyT>;
  constexpr int PASSES = KT::PASSES;
  constexpr int NW     = KT::NWORDS;
  using DT             = DigitThreads<BLOCK>;
  using SW             = unsigned long long;  // a key's digits, eight to a word, as shuffled across the wave
  using IdxS           = uint16_t;  // row position while staged in LDS
  static_assert(TILE <= 65536, "row positions are staged as 16 bits");
  // not for 2-byte keys (their codec is cheap) nor for 1024 threads: there the second code path
  // costs registers beyond the 64 that let two workgroups share a CU
  constexpr bool IMAGES_OK = (CODEC == CODEC_FLOAT) && sizeof(KeyT) >= 4 && BLOCK <= 512;

  // the split on leading bits: real keys of 4 and 8 bytes, values only
  // (only the 1024-thread shapes, rows of more than 4096 keys: in the smaller shapes the bins cost
  // the LDS that lets many workgroups share a CU, and rows of 1024 float64 keys went from 0.41 to 0.60 ms)
  // (every shape of at least four keys per thread: measured on 2^26 keys, passes / split: rows of 1024 float64 0.35 / 0.30 ms,
  // 2048 float64 0.47 / 0.34, 4096 float64 0.50 / 0.37, 1500 float32 0.48 / 0.30, 2048 float32 0.36 / 0.25,
  // 4096 int32 0.35 / 0.30; with positions 2048 float32 0.43 / 0.32, 2048 float64 0.55 / 0.40 ms)
  constexpr bool BUCKETS_SHAPE = BLOCK >= 64 && ITEMS >= 4;  // (64 x 4 ... 64 x 12: one wavefront per row of up to 768 keys)
  constexpr bool BUCKETS_OK = NW == 1 && sizeof(KeyT) >= 4 && sizeof(KeyT) <= 8 && BUCKETS_SHAPE &&
                              (CODEC == CODEC_UNSIGNED || CODEC == CODEC_SIGNED || CODEC == CODEC_FLOAT);
  constexpr int BINS_LOG2   = bucket_bins_log2(TILE, sizeof(KeyT), HAS_IDX, BLOCK);
  constexpr int BINS        = 1 << BINS_LOG2;
  constexpr int BINS_PER_THREAD = BINS / BLOCK;
  static_assert(!BUCKETS_OK || (BINS_PER_THREAD >= 4 && BINS_PER_THREAD % 4 == 0), "a thread scans whole 16-byte chunks");

  // (padded where the split is compiled in: its walk over a bin reads up to BUCKET_LIMIT keys past the bin's end)
  __shared__ __align__(16) KeyT s_keys[TILE + (BUCKETS_OK ? BUCKET_PAD : 0)];
  __shared__ IdxS s_idx[HAS_IDX ? TILE + (BUCKETS_OK ? BUCKET_PAD : 0) : 1];
  // the per-wave digit counters of the radix passes and the bins of the split share their memory
  // (the split is over, or given up, before the first radix pass clears its counters)
  constexpr int CTR_WORDS = (BUCKETS_OK && BINS > WAVES * RADIX) ? BINS : WAVES * RADIX;
  __shared__ __align__(16) uint32_t s_ctr[CTR_WORDS];
  uint32_t* const s_bins = s_ctr;
  __shared__ uint32_t s_wsum[DT::WAVES];
  __shared__ SW s_red[2 * WAVES * NW];

  const int tid       = threadIdx.x;
  const int lane      = tid & (WAVE - 1);
  const int wave      = tid / WAVE;
  // A workgroup sorts one piece of a row: the whole row (pieces == 1; row_stride == piece_len where the
  // rows are dense), or, for rows that are merged afterwards, piece number blockIdx.x % pieces of row
  // blockIdx.x / pieces; the last piece of a row may be shorter, and positions count from the row's start.
  uint32_t seg  = piece_len;
  uint64_t base = static_cast<uint64_t>(blockIdx.x) * row_stride;
  if (pieces > 1) {
    const uint32_t row   = blockIdx.x / pieces;
    const uint32_t piece = blockIdx.x - row * pieces;
    base                 = static_cast<uint64_t>(row) * row_stride + static_cast<uint64_t>(piece) * piece_len;
    index_offset += static_cast<int64_t>(piece) * piece_len;
    seg = piece + 1 == pieces ? last_piece_len : piece_len;
  }
  const bool full     = (seg == TILE);
  // A row shorter than the tile is dealt in equal contiguous shares of whole 64-key rounds, so that
  // every wave works on `rounds` keys per lane and the cost follows the row length, not the tile.
  // (Only the 1024-thread shapes, which take the longest rows and a wide range of lengths: in the
  // smaller ones the extra uniform branches cost full rows 3-10 % and the shapes are a factor of two apart.)
  constexpr bool BALANCE = (BLOCK == 1024);
  const uint32_t rounds  = (!BALANCE || full) ? ITEMS : (seg + BLOCK - 1) / BLOCK;
  const uint32_t woff    = wave * ((!BALANCE || full) ? WTILE : rounds * WAVE) + lane;
  auto holds = [&](int i) -> bool {
    return full || ((!BALANCE || i < static_cast<int>(rounds)) && woff + i * WAVE < seg);
  };

  KeyT key[ITEMS];
  uint32_t idx[HAS_IDX ? ITEMS : 1];
  // (all loads first, from offsets that are inside the row whatever the lane holds, so that none of
  // them sits behind a branch and waits for the one before it; one uniform row pointer and 32-bit
  // offsets, so that the addresses of 16 loads in flight do not take 32 registers)
  const KeyT* const row_in = keys_in + base;
#pragma unroll
  for (int i = 0; i < ITEMS; ++i) {
    const uint32_t o = woff + i * WAVE;
    key[i]           = row_in[o < seg ? o : seg - 1];
    if constexpr (HAS_IDX) {
      idx[i] = o;
    }
  }
  // ---- bits on which the keys of the row differ (passes on the other digits are skipped), and for
  //      float keys whether the row holds a NaN or a -0.0 ----
  // Real keys: taken from the keys' own bits.  The ordered image of a signed integer, and of a float
  // row whose keys share one sign and hold no NaN and no -0.0, is the key XOR a constant, so it varies
  // in the same bits; any other float row is taken to vary in every bit (it nearly always does: the
  // images of its negative keys are complemented).  Complex keys: from the words of the image.
  constexpr bool RAW_BITS = (NW == 1) && (CODEC == CODEC_UNSIGNED || CODEC == CODEC_SIGNED || CODEC == CODEC_FLOAT);
  SW all_and[NW], all_or[NW];
  int special = 0;  // float keys: the row holds a NaN or a -0.0
#pragma unroll
  for (int n = 0; n < NW; ++n) {
    all_and[n] = ~static_cast<SW>(0);
    all_or[n]  = 0;
  }
  if constexpr (RAW_BITS) {
    KeyT bits_and = static_cast<KeyT>(~static_cast<KeyT>(0)), bits_or = 0;
#pragma unroll
    for (int i = 0; i < ITEMS; ++i) {
      if (holds(i)) {
        bits_and &= key[i];
        bits_or |= key[i];
        if constexpr (CODEC == CODEC_FLOAT) {
          special |= is_nan_or_negative_zero(key[i]) ? 1 : 0;
        }
      } else {
        key[i] = KeyT{};
      }
    }
    all_and[0] = static_cast<SW>(bits_and);
    all_or[0]  = static_cast<SW>(bits_or);
  } else {
#pragma unroll
    for (int i = 0; i < ITEMS; ++i) {
      if (holds(i)) {
        uint64_t w[NW];
        KT::words(key[i], w);
#pragma unroll
        for (int n = 0; n < NW; ++n) {
          all_and[n] &= w[n];
          all_or[n] |= w[n];
        }
        if constexpr (CODEC == CODEC_FLOAT) {
          special |= (static_cast<KeyT>(w[0]) != sign_flip(key[i])) ? 1 : 0;
        }
      } else {
        key[i] = KeyT{};
      }
    }
  }
  using RedT = typename std::conditional<(sizeof(KeyT) <= 4 && NW == 1), uint32_t, SW>::type;  // the half that can be set
#pragma unroll
  for (int n = 0; n < NW; ++n) {
    all_and[n] = wave_reduce_and_dpp(static_cast<RedT>(all_and[n]));
    all_or[n]  = wave_reduce_or_dpp(static_cast<RedT>(all_or[n]));
    if (lane == 0) {
      s_red[(2 * wave) * NW + n]     = all_and[n];
      s_red[(2 * wave + 1) * NW + n] = all_or[n];
    }
  }
  const int any_special = __syncthreads_or(special);
  bool images           = IMAGES_OK && (any_special == 0);
  // Sorts that return keys only: the first pass to run need not be stable.  Keys that tie in every
  // digit are the same bits (float rows with a NaN or a -0.0, where different bits tie, are left
  // out; so are complex keys), so nothing shows in which order that pass leaves equal digits, and
  // every later pass is stable.  Its ranks then come from one LDS atomic per key on counters
  // shared by the workgroup instead of the ballots of the stable ranking.
  const bool free_first = !HAS_IDX && (CODEC == CODEC_UNSIGNED || CODEC == CODEC_SIGNED ||
                                       (CODEC == CODEC_FLOAT && any_special == 0));
  bool first_running    = true;
  SW varying[NW];
#pragma unroll
  for (int n = 0; n < NW; ++n) {
    SW a, o;
    if constexpr (WAVES >= 8) {
      // every lane takes the words of one wave; AND and OR do not mind seeing a wave several times
      a = wave_reduce_and_dpp(static_cast<RedT>(s_red[(2 * (lane % WAVES)) * NW + n]));
      o = wave_reduce_or_dpp(static_cast<RedT>(s_red[(2 * (lane % WAVES) + 1) * NW + n]));
    } else {
      a = s_red[n], o = s_red[NW + n];
#pragma unroll
      for (int w = 1; w < WAVES; ++w) {
        a &= s_red[(2 * w) * NW + n];
        o |= s_red[(2 * w + 1) * NW + n];
      }
    }
    varying[n] = a ^ o;
  }
  if constexpr (RAW_BITS && CODEC == CODEC_FLOAT) {
    constexpr SW SIGN = static_cast<SW>(1) << (8 * sizeof(KeyT) - 1);
    if (any_special != 0 || (varying[0] & SIGN) != 0) {
      varying[0] = ~static_cast<SW>(0);
    }
  }
  uint32_t active = 0;  // bit p: the keys of the row differ in digit p
#pragma unroll
  for (int p = 0; p < PASSES; ++p) {
    if (((varying[p / 8] >> ((p % 8) * RADIX_BITS)) & 0xFFu) != 0) {
      active |= 1u << p;
    }
  }

  // leading-digits shortcut (see the head of this file)
  uint32_t todo  = active;
  bool shortcut  = false;
  if constexpr (PASSES >= 5) {
    const int lead = (2 * (32 - __builtin_clz(seg - 1 | 1u)) + 4 + RADIX_BITS - 1) / RADIX_BITS;
    if (__builtin_popcount(active) >= lead + 2) {
      uint32_t rem = active;
      todo         = 0;
      for (int t = 0; t < lead; ++t) {
        const uint32_t top = 1u << (31 - __builtin_clz(rem));
        todo |= top;
        rem ^= top;
      }
      shortcut = true;
    }
  }

  uint32_t* wctr = s_ctr + wave * RADIX;
  // float rows held as images take plain bytes; `images` is uniform, so the choice is a scalar branch
  auto digit_of = [&](KeyT k, int pass) -> uint32_t {
    if constexpr (IMAGES_OK) {
      if (images) {
        return KeyTraits<CODEC_UNSIGNED, KeyT>::digit(k, pass);
      }
    }
    return KT::digit(k, pass);
  };
  auto words_of = [&](KeyT k, uint64_t (&w)[NW]) {
    if constexpr (IMAGES_OK) {
      if (images) {
        w[0] = static_cast<uint64_t>(k);
        return;
      }
    }
    KT::words(k, w);
  };
  if constexpr (BUCKETS_OK) {
    // Sorts that carry positions take the split too: a key's place inside its bin then counts the
    // smaller keys and the equal ones of lower position, which is the stable order; the keys' own
    // comparison has to be the sort order, so float rows with a NaN or a -0.0 stay out here as well.
    const bool split_ok = HAS_IDX ? (CODEC != CODEC_FLOAT || any_special == 0) : free_first;
    if (split_ok && __builtin_popcount(active) >= 2) {  // uniform
      using NT = typename NativeKey<CODEC, sizeof(KeyT)>::type;  // float, double or the integer type
      auto native = [](KeyT k) -> NT {
        NT v;
        __builtin_memcpy(&v, &k, sizeof(NT));
        return v;
      };
      // (no NaN among the keys: the float minimum and maximum instructions order them like `<`)
      auto lower = [](NT a, NT b) -> NT {
        if constexpr (std::is_same<NT, float>::value) {
          return __builtin_fminf(a, b);
        } else if constexpr (std::is_same<NT, double>::value) {
          return __builtin_fmin(a, b);
        } else {
          return a < b ? a : b;
        }
      };
      auto upper = [](NT a, NT b) -> NT {
        if constexpr (std::is_same<NT, float>::value) {
          return __builtin_fmaxf(a, b);
        } else if constexpr (std::is_same<NT, double>::value) {
          return __builtin_fmax(a, b);
        } else {
          return a > b ? a : b;
        }
      };
      // smallest and largest key of the row (the row holds no NaN and no -0.0: the keys' own order
      // is the sort order), through the staging area, which is free until the keys are placed
      NT lo = std::numeric_limits<NT>::max(), hi = std::numeric_limits<NT>::lowest();  // (lanes that hold no key)
#pragma unroll
      for (int i = 0; i < ITEMS; ++i) {
        if (holds(i)) {
          const NT v = native(key[i]);
          lo         = lower(v, lo);
          hi         = upper(v, hi);
        }
      }
#pragma unroll
      for (int d = 1; d < WAVE; d <<= 1) {
        lo = lower(__shfl_xor(lo, d, WAVE), lo);
        hi = upper(__shfl_xor(hi, d, WAVE), hi);
      }
      NT* s_ext = reinterpret_cast<NT*>(s_keys);
      if (lane == 0) {
        s_ext[wave]         = lo;
        s_ext[WAVES + wave] = hi;
      }
      for (int j = tid; j < BINS / 4; j += BLOCK) {
        reinterpret_cast<uint4*>(s_bins)[j] = make_uint4(0u, 0u, 0u, 0u);
      }
      __syncthreads();
      // (every lane takes the extremes of one wave, four exchanges inside each group of 16 lanes
      // merge them; minimum and maximum do not mind seeing a wave several times)
      static_assert(WAVES <= WAVE && (WAVES & (WAVES - 1)) == 0, "one wave per lane of a group of WAVES lanes");
      lo = s_ext[lane % WAVES];
      hi = s_ext[WAVES + lane % WAVES];
#pragma unroll
      for (int d = 1; d < WAVES; d <<= 1) {
        lo = lower(__shfl_xor(lo, d, WAVE), lo);
        hi = upper(__shfl_xor(hi, d, WAVE), hi);
      }
      // The bin of a key: its place between the smallest and the largest key, in equal steps of the
      // value.  Float keys: subtraction of a constant, scaling and truncation never decrease with the
      // key, rounding included, so a key in a lower bin is a smaller key, which is all the split
      // needs.  (An infinite extreme or span makes the scale 0 or the product NaN, which is clamped to
      // bin 0: the row then crowds one bin and takes the radix passes.)  Integer keys: the distance
      // from the smallest key, shifted down until the largest distance fits the bins.
      using FT = typename std::conditional<sizeof(KeyT) == 4, float, double>::type;
      FT origin = 0, scale = 0;
      KeyT img_lo = 0;
      int shift   = 0;
      if constexpr (CODEC == CODEC_FLOAT) {
        origin = lo;
        scale  = static_cast<FT>(BINS) / (hi - lo);
      } else {
        img_lo          = ordered_bits<CODEC, KeyT>(static_cast<KeyT>(lo));
        const KeyT span = static_cast<KeyT>(ordered_bits<CODEC, KeyT>(static_cast<KeyT>(hi)) - img_lo);
        const int bits  = 64 - __builtin_clzll(static_cast<unsigned long long>(span) | 1ull);
        shift           = bits > BINS_LOG2 ? bits - BINS_LOG2 : 0;
      }
      auto bin_of = [&](KeyT k) -> uint32_t {
        if constexpr (CODEC == CODEC_FLOAT) {
          // (clamped as a floating-point value before the conversion, which is undefined for NaN and
          // out-of-range values; fmax returns its other operand for a NaN)
          FT t = (native(k) - origin) * scale;
          if constexpr (sizeof(FT) == 4) {
            t = __builtin_fminf(__builtin_fmaxf(t, 0.0f), static_cast<float>(BINS - 1));
          } else {
            t = __builtin_fmin(__builtin_fmax(t, 0.0), static_cast<double>(BINS - 1));
          }
          return static_cast<uint32_t>(t);
        } else {
          return static_cast<uint32_t>(static_cast<KeyT>(ordered_bits<CODEC, KeyT>(k) - img_lo) >> shift);
        }
      };
      // (a partly filled tile: rounds in which no wave holds a key are skipped as a whole)
      auto round_runs = [&](int i) -> bool { return !BALANCE || full || i < static_cast<int>(rounds); };
      uint32_t bin[ITEMS];
#pragma unroll
      for (int i = 0; i < ITEMS; ++i) {
        bin[i] = 0;
        if (round_runs(i)) {  // uniform
          bin[i] = bin_of(key[i]);
          if (holds(i)) {
            atomicAdd(&s_bins[bin[i]], 1u);
          }
        }
      }
      __syncthreads();
      // exclusive scan of the bins: thread t owns bins [t*BINS_PER_THREAD, (t+1)*BINS_PER_THREAD)
      uint32_t cnt[BINS_PER_THREAD];
      uint32_t total = 0, largest = 0;
#pragma unroll
      for (int c = 0; c < BINS_PER_THREAD / 4; ++c) {
        const uint4 q4 = *reinterpret_cast<const uint4*>(&s_bins[tid * BINS_PER_THREAD + 4 * c]);
        cnt[4 * c] = q4.x, cnt[4 * c + 1] = q4.y, cnt[4 * c + 2] = q4.z, cnt[4 * c + 3] = q4.w;
      }
#pragma unroll
      for (int j = 0; j < BINS_PER_THREAD; ++j) {
        total += cnt[j];
        largest = cnt[j] > largest ? cnt[j] : largest;
      }
      const uint32_t incl = wave_inclusive_sum_dpp(total);
      if (lane == WAVE - 1) {
        s_wsum[wave] = incl;
      }
      constexpr uint32_t LIMIT = (TILE > 2 * BINS) ? BUCKET_LIMIT_WIDE : BUCKET_LIMIT;
      static_assert(LIMIT <= static_cast<uint32_t>(BUCKET_PAD), "the walk reads up to LIMIT keys past a bin's end");
      const int crowded = __syncthreads_or(largest > LIMIT ? 1 : 0);
      if (crowded == 0) {
        uint32_t run = incl - total;
        for (int w = 0; w < wave; ++w) {
          run += s_wsum[w];
        }
#pragma unroll
        for (int c = 0; c < BINS_PER_THREAD / 4; ++c) {
          uint32_t e[4];
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            e[j] = run;
            run += cnt[4 * c + j];
          }
          *reinterpret_cast<uint4*>(&s_bins[tid * BINS_PER_THREAD + 4 * c]) = make_uint4(e[0], e[1], e[2], e[3]);
        }
        __syncthreads();
        // every key into its bin, in whatever order the atomics hand out
        // (without positions a key remembers where it went: that breaks the ties of the walk below;
        // with positions the positions do, and the registers are needed elsewhere)
        uint32_t self[HAS_IDX ? 1 : ITEMS];
#pragma unroll
        for (int i = 0; i < ITEMS; ++i) {
          if constexpr (!HAS_IDX) {
            self[i] = 0;
          }
          if (round_runs(i) && holds(i)) {
            const uint32_t went = atomicAdd(&s_bins[bin[i]], 1u);
            s_keys[went]        = key[i];
            if constexpr (HAS_IDX) {
              s_idx[went] = static_cast<IdxS>(idx[i]);
            } else {
              self[i] = went;
            }
          }
        }
        __syncthreads();
        // Each bin now ends where its counter stands and starts where the bin before it ends.  A key
        // goes to the start of its bin plus the number of keys of the bin that come before it: smaller
        // ones, and equal ones that the atomics placed earlier (equal keys are the same bits here, the
        // rule only keeps the places distinct).
        // (Eight keys of a thread walk their bins in step, so that every round has eight independent
        // LDS reads in flight instead of one; a read past the end of a bin fetches a key of a later
        // bin, or of the padding, and is not counted.  Eight at a time, not all: the walk's state for
        // 16 keys does not fit the registers of a 1024-thread workgroup.)
        // (with positions: ties go by the position the key came from, read from LDS beside the key, and
        // four keys walk at a time)
        constexpr int GROUP = HAS_IDX ? (ITEMS % 4 == 0 ? 4 : 2) : (ITEMS < 8 ? ITEMS : (ITEMS % 8 == 0 ? 8 : (ITEMS % 4 == 0 ? 4 : 2)));
        static_assert(ITEMS % GROUP == 0, "whole groups");
#pragma unroll
        for (int g = 0; g < ITEMS; g += GROUP) {
          if (!round_runs(g)) {
            continue;  // uniform: no wave holds a key of this group
          }
          uint32_t from[GROUP], len[GROUP], before[GROUP];
          uint32_t longest = 0;
#pragma unroll
          for (int k = 0; k < GROUP; ++k) {
            const int i = g + k;
            from[k] = 0, len[k] = 0, before[k] = 0;
            if (round_runs(i) && holds(i)) {
              const uint32_t end = s_bins[bin[i]];
              from[k]            = (bin[i] == 0) ? 0u : s_bins[bin[i] - 1];  // start of the bin
              len[k]             = end - from[k];
              if constexpr (!HAS_IDX) {
                self[i] -= from[k];
              }
              longest = len[k] > longest ? len[k] : longest;
            }
          }
          // (two copies of the loop: a group whose every round runs pays no per-round checks)
          auto walk = [&](auto every_round) {
            for (uint32_t j = 0; j < longest; ++j) {
              KeyT other[GROUP];
              uint32_t other_idx[HAS_IDX ? GROUP : 1];
#pragma unroll
              for (int k = 0; k < GROUP; ++k) {
                if (!decltype(every_round)::value && !round_runs(g + k)) {
                  break;
                }
                other[k] = s_keys[from[k] + j];
                if constexpr (HAS_IDX) {
                  other_idx[k] = s_idx[from[k] + j];
                }
              }
#pragma unroll
              for (int k = 0; k < GROUP; ++k) {
                if (!decltype(every_round)::value && !round_runs(g + k)) {
                  break;
                }
                const NT a = native(other[k]), b = native(key[g + k]);
                // (bitwise, not short-circuit: no branch between the reads of a round)
                bool first;
                if constexpr (HAS_IDX) {
                  first = (a < b) | ((a == b) & (other_idx[k] < idx[g + k]));
                } else {
                  first = (a < b) | ((a == b) & (j < self[g + k]));
                }
                before[k] += (first & (j < len[k])) ? 1u : 0u;
              }
            }
          };
          if (round_runs(g + GROUP - 1)) {
            walk(std::true_type{});
          } else {
            walk(std::false_type{});
          }
#pragma unroll
          for (int k = 0; k < GROUP; ++k) {
            bin[g + k] = from[k] + before[k];  // where the key belongs (its bin number is no longer needed)
          }
        }
        __syncthreads();
#pragma unroll
        for (int i = 0; i < ITEMS; ++i) {
          if (round_runs(i) && holds(i)) {
            s_keys[bin[i]] = key[i];
            if constexpr (HAS_IDX) {
              s_idx[bin[i]] = static_cast<IdxS>(idx[i]);
            }
          }
        }
        __syncthreads();
#pragma unroll
        for (int i = 0; i < ITEMS; ++i) {
          if (holds(i)) {
            key[i] = s_keys[woff + i * WAVE];
            if constexpr (HAS_IDX) {
              idx[i] = s_idx[woff + i * WAVE];
            }
          }
        }
        todo     = 0;      // sorted: no radix pass is left
        shortcut = false;
      }
    }
  }
  // (after the split, which works on the keys' own bits; a row that the split has sorted needs no images)
  images = images && todo != 0;
  if constexpr (IMAGES_OK) {
    if (images) {
#pragma unroll
      for (int i = 0; i < ITEMS; ++i) {
        key[i] = sign_flip(key[i]);
      }
    }
  }
  for (;;) {
  for (int pass = 0; pass < PASSES; ++pass) {
    if (((todo >> pass) & 1u) == 0) {
      continue;  // uniform for the block
    }
    for (int j = tid; j < WAVES * RADIX; j += BLOCK) {
      s_ctr[j] = 0;
    }
    __syncthreads();
    uint32_t rnk[ITEMS];
    uint32_t dpk[(ITEMS + 3) / 4];  // the digits, four per register
#pragma unroll
    for (int i = 0; i < ITEMS; ++i) {
      if constexpr (BALANCE) {
        if (!full && i >= static_cast<int>(rounds)) {
          break;  // uniform: no wave holds a key in this round
        }
      }
      const bool valid = holds(i);
      const uint32_t d = digit_of(key[i], pass);
      dpk[i / 4]       = (i % 4 == 0) ? d : (dpk[i / 4] | (d << (8 * (i % 4))));
      if (!HAS_IDX && free_first && first_running) {  // uniform
        rnk[i] = valid ? atomicAdd(&s_ctr[d], 1u) : 0u;  // wave 0's counters serve the whole workgroup
      } else {
        rnk[i] = wave_match_rank(d, valid, wctr);
      }
    }
    const uint32_t* base = (!HAS_IDX && free_first && first_running) ? s_ctr : wctr;
    first_running        = false;
    __syncthreads();
    // exclusive scan over (digit, wave) in digit-major order
    uint32_t tsum = 0, tincl = 0;
    if (tid < DT::THREADS) {
#pragma unroll
      for (int j = 0; j < DT::PER_THREAD; ++j) {
        const int d = tid * DT::PER_THREAD + j;
#pragma unroll
        for (int w = 0; w < WAVES; ++w) {
          const uint32_t c     = s_ctr[w * RADIX + d];
          s_ctr[w * RADIX + d] = tsum;
          tsum += c;
        }
      }
      tincl = wave_inclusive_scan(tsum, lane);
      if (lane == WAVE - 1) {
        s_wsum[wave] = tincl;
      }
    }
    __syncthreads();
    if (tid < DT::THREADS) {
      uint32_t texcl = tincl - tsum;
      for (int w = 0; w < wave; ++w) {
        texcl += s_wsum[w];
      }
#pragma unroll
      for (int j = 0; j < DT::PER_THREAD; ++j) {
        const int d = tid * DT::PER_THREAD + j;
#pragma unroll
        for (int w = 0; w < WAVES; ++w) {
          s_ctr[w * RADIX + d] += texcl;
        }
      }
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < ITEMS; ++i) {
      if (holds(i)) {
        const uint32_t d   = (dpk[i / 4] >> (8 * (i % 4))) & 0xFFu;
        const uint32_t pos = base[d] + rnk[i];
        s_keys[pos]        = key[i];
        if constexpr (HAS_IDX) {
          s_idx[pos] = static_cast<IdxS>(idx[i]);
        }
      }
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < ITEMS; ++i) {
      const uint32_t o = woff + i * WAVE;
      if (holds(i)) {
        key[i] = s_keys[o];
        if constexpr (HAS_IDX) {
          idx[i] = s_idx[o];
        }
      }
    }
    // the next pass (or nothing) touches s_keys only after its own barriers
  }
    if (!shortcut) {
      break;
    }
    // s_keys holds the row as ordered by the leading digits: is every neighbouring pair in order?
    // A few pairs that are not (keys that tie on the leading digits) are put right by rounds of
    // odd-even transposition in LDS, which exchanges strictly misordered neighbours only and so
    // keeps equal keys in input order.
    auto misordered = [&](KeyT first, KeyT second) -> bool {
      uint64_t a[NW], b[NW];
      words_of(first, a);
      words_of(second, b);
      bool gt = false, eq = true;  // a > b, most significant word first
#pragma unroll
      for (int n = NW - 1; n >= 0; --n) {
        gt = gt || (eq && a[n] > b[n]);
        eq = eq && (a[n] == b[n]);
      }
      return gt;
    };
    bool in_order = false;
    for (int round = 0;; ++round) {
      int bad = 0;
#pragma unroll
      for (int i = 0; i < ITEMS; ++i) {
        const uint32_t o = woff + i * WAVE;
        if (holds(i) && o + 1 < seg) {
          bad |= misordered(key[i], s_keys[o + 1]) ? 1 : 0;
        }
      }
      if (__syncthreads_or(bad) == 0) {
        in_order = true;
        break;
      }
      if (round == FIXUP_ROUNDS) {
        break;
      }
      for (uint32_t phase = 0; phase < 2; ++phase) {
        for (uint32_t p = 2 * tid + phase; p + 1 < seg; p += 2 * BLOCK) {
          const KeyT first = s_keys[p], second = s_keys[p + 1];
          if (misordered(first, second)) {
            s_keys[p]     = second;
            s_keys[p + 1] = first;
            if constexpr (HAS_IDX) {
              const IdxS t = s_idx[p];
              s_idx[p]     = s_idx[p + 1];
              s_idx[p + 1] = t;
            }
          }
        }
        __syncthreads();
      }
#pragma unroll
      for (int i = 0; i < ITEMS; ++i) {
        const uint32_t o = woff + i * WAVE;
        if (holds(i)) {
          key[i] = s_keys[o];
          if constexpr (HAS_IDX) {
            idx[i] = s_idx[o];
          }
        }
      }
    }
    if (in_order) {
      break;
    }
    shortcut = false;
    todo     = active;
  }
  if constexpr (IMAGES_OK) {
    if (images) {
#pragma unroll
      for (int i = 0; i < ITEMS; ++i) {
        key[i] = sign_unflip(key[i]);
      }
    }
  }

#pragma unroll
  for (int i = 0; i < ITEMS; ++i) {
    const uint32_t o = woff + i * WAVE;
    if (holds(i)) {
      if (keys_out != nullptr) {
        keys_out[base + o] = key[i];
      }
      if constexpr (HAS_IDX) {
        idx_out[base + o] = static_cast<int64_t>(idx[i]) + index_offset;
      }
    }
  }
}

}  // namespace cpn
