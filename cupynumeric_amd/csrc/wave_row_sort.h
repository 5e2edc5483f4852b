// Short rows (up to 1024 elements): one wavefront sorts one row, several rows per workgroup,
// and no workgroup barrier anywhere -- the 64 lanes of a wave execute their LDS operations in
// order, so the phases of a pass need no synchronisation beyond that.
//
// The keys are turned into their order-preserving unsigned words once, when they are loaded,
// and stay in registers in that form: a pass only extracts a byte.  Integer keys are mapped
// back at the end (the transform is a bijection); float and complex keys cannot be (-0.0 and
// NaN payloads are folded), so those rows always carry the 16-bit source position along and
// the sorted values are gathered from the input row by position after the last pass.
//
// Replaces, for such rows, the (segment id, value) tuple merge sort of
// src/cupynumeric/sort/thrust_sort.cuh:68-122 (rows of at most 400 elements) and
// cub::DeviceSegmentedRadixSort (src/cupynumeric/sort/cub_sort.cuh:81-105,153-182).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "radix_common.h"

namespace cpn {

// odd-even transposition rounds tried after the leading-digit shortcut of the row kernels
constexpr int FIXUP_ROUNDS = 4;

// The ordered key of one element as 32-bit words, least significant first; digit p is byte
// p%4 of word p/4.
template <int CODEC, typename KeyT>
struct OrderedWords {
  using KT                     = KeyTraits<CODEC, KeyT>;
  static constexpr int PASSES  = KT::PASSES;
  static constexpr int NW      = (PASSES + 3) / 4;
  static constexpr bool BIJECT = (CODEC == CODEC_UNSIGNED || CODEC == CODEC_SIGNED);

  static __device__ __forceinline__ void encode(KeyT raw, uint32_t (&w)[NW])
  {
    uint64_t q[KT::NWORDS];
    KT::words(raw, q);
#pragma unroll
    for (int n = 0; n < NW; ++n) {
      w[n] = static_cast<uint32_t>(q[n / 2] >> ((n % 2) * 32));
    }
  }
  // float keys that are neither NaN nor -0.0: the image determines the bits
  static __device__ __forceinline__ KeyT decode_plain_float(const uint32_t (&w)[NW])
  {
    if constexpr (CODEC == CODEC_FLOAT && sizeof(KeyT) <= 8) {
      uint64_t v = w[0];
      if constexpr (NW > 1) {
        v |= static_cast<uint64_t>(w[1]) << 32;
      }
      return sign_unflip(static_cast<KeyT>(v));
    } else {
      return KeyT{};
    }
  }
  // only for bijective codecs
  static __device__ __forceinline__ KeyT decode(const uint32_t (&w)[NW])
  {
    if constexpr (sizeof(KeyT) <= 8 && BIJECT) {
      uint64_t v = w[0];
      if constexpr (NW > 1) {
        v |= static_cast<uint64_t>(w[1]) << 32;
      }
      const KeyT o = static_cast<KeyT>(v);
      if constexpr (CODEC == CODEC_SIGNED) {
        return static_cast<KeyT>(o ^ (static_cast<KeyT>(1) << (sizeof(KeyT) * 8 - 1)));
      } else {
        return o;
      }
    } else {
      return KeyT{};
    }
  }
};

template <typename T>
__device__ __forceinline__ T wave_all_and(T v)
{
#pragma unroll
  for (int delta = WAVE / 2; delta > 0; delta >>= 1) {
    v &= __shfl_xor(v, delta, WAVE);
  }
  return v;
}
template <typename T>
__device__ __forceinline__ T wave_all_or(T v)
{
#pragma unroll
  for (int delta = WAVE / 2; delta > 0; delta >>= 1) {
    v |= __shfl_xor(v, delta, WAVE);
  }
  return v;
}

// Sorts of real 4-byte keys whose ties are the same bits (integers; floats without NaN and -0.0) or
// whose ties can go by the position carried with every key (argsort) need no stable passes: the row is split into ranges of equal width between its smallest
// and largest key, two per key, with one LDS atomic per key, and every key then counts the smaller
// keys of its range (the same idea as in the one-workgroup-per-row kernel, lds_row_sort.h, here
// within one wave and without any barrier).  A row that crowds a range takes the radix passes.
// Measured on 2^26 .. 2^28 float32 keys, radix passes / split: rows of 64 0.53 / 0.45 ms, 128 1.63 / 1.42,
// 256 0.33 / 0.28, 512 0.36 / 0.28, 1024 0.37 / 0.46 ms: rows of up to 512 keys take it.
template <int CODEC, typename KeyT, bool HAS_IDX, int ITEMS>
__host__ __device__ constexpr bool wave_split_ok()
{
  (void)HAS_IDX;  // with positions too: ties inside a range then go by position, the stable order
  return sizeof(KeyT) == 4 && ITEMS <= 8 && (CODEC == CODEC_UNSIGNED || CODEC == CODEC_SIGNED || CODEC == CODEC_FLOAT);
}
// ranges (bins) of the split for a tile of `tile` keys; their counters share the memory of the
// 256 digit counters of the radix passes
__host__ __device__ constexpr int wave_split_bins(int tile) { return 2 * tile > RADIX ? 2 * tile : RADIX; }
constexpr uint32_t WAVE_SPLIT_LIMIT = 12;  // most keys a range may hold

// bytes of LDS one wave (= one row) needs
template <int CODEC, typename KeyT, int ITEMS, bool HAS_IDX = true>
__host__ __device__ constexpr int wave_row_lds_bytes()
{
  return OrderedWords<CODEC, KeyT>::NW * 4 * ITEMS * WAVE + 2 * ITEMS * WAVE +
         (wave_split_ok<CODEC, KeyT, HAS_IDX, ITEMS>() ? wave_split_bins(ITEMS * WAVE) : RADIX) * 4;
}

template <typename KeyT, int CODEC, bool HAS_IDX, int ITEMS, int ROWS_PER_BLOCK>
__global__ __launch_bounds__(WAVE* ROWS_PER_BLOCK) void wave_row_sort_kernel(const KeyT* keys_in,
                                                                              KeyT* keys_out,
                                                                              int64_t* idx_out,
                                                                              uint32_t seg,
                                                                              uint64_t rows,
                                                                              int64_t index_offset,
                                                                              uint32_t* status)
{
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    *status = 0;  // the workspace's status word: a per-row sort cannot fail on the device
  }
  using OW                = OrderedWords<CODEC, KeyT>;
  constexpr int NW        = OW::NW;
  constexpr int PASSES    = OW::PASSES;
  constexpr int TILE      = ITEMS * WAVE;
  // Float keys without indices: the sorted images give back every key but NaNs and zeros, whose
  // bits the image does not hold; those are put in place at the end from a second look at the input.
  constexpr bool FLOAT_KEYS_ONLY = (CODEC == CODEC_FLOAT) && !HAS_IDX && sizeof(KeyT) <= 8;
  constexpr bool CARRY           = HAS_IDX || !(OW::BIJECT || FLOAT_KEYS_ONLY);  // source positions travel with the keys
  static_assert(TILE <= 65536, "positions are 16 bits");

  __shared__ uint32_t s_words[ROWS_PER_BLOCK][NW][TILE];
  __shared__ uint16_t s_pos[ROWS_PER_BLOCK][CARRY ? TILE : 1];
  constexpr bool SPLIT_OK = wave_split_ok<CODEC, KeyT, HAS_IDX, ITEMS>();
  constexpr int BINS      = SPLIT_OK ? wave_split_bins(TILE) : RADIX;
  __shared__ __align__(16) uint32_t s_ctr[ROWS_PER_BLOCK][BINS];

  const int lane     = threadIdx.x & (WAVE - 1);
  const int wave     = threadIdx.x / WAVE;
  const uint64_t row = static_cast<uint64_t>(blockIdx.x) * ROWS_PER_BLOCK + wave;
  if (row >= rows) {
    return;  // whole wave; no workgroup barrier is used below
  }
  const uint64_t base = row * seg;
  uint32_t* ctr       = s_ctr[wave];
  const bool full     = (seg == TILE);

  // ---- load, item i of lane l is element i*64 + l of the row; encode once ----
  uint32_t w[ITEMS][NW];
  uint32_t pos2[CARRY ? (ITEMS + 1) / 2 : 1];  // source positions, two per register
  uint32_t vary_and[NW], vary_or[NW];
  bool special = false;  // float keys: a NaN or a -0.0 (different bits that tie)
#pragma unroll
  for (int n = 0; n < NW; ++n) {
    vary_and[n] = 0xFFFFFFFFu;
    vary_or[n]  = 0;
  }
  // (all loads first, from addresses that are inside the row whatever the lane holds, so that none
  // of them sits behind a branch and waits for the one before it)
  KeyT loaded[ITEMS];
#pragma unroll
  for (int i = 0; i < ITEMS; ++i) {
    const uint32_t o = i * WAVE + lane;
    loaded[i]        = keys_in[base + (o < seg ? o : seg - 1)];
  }
#pragma unroll
  for (int i = 0; i < ITEMS; ++i) {
    const uint32_t o = i * WAVE + lane;
    if (full || o < seg) {
      const KeyT raw = loaded[i];
      OW::encode(raw, w[i]);
#pragma unroll
      for (int n = 0; n < NW; ++n) {
        vary_and[n] &= w[i][n];
        vary_or[n] |= w[i][n];
      }
      if constexpr (CODEC == CODEC_FLOAT && (!HAS_IDX || wave_split_ok<CODEC, KeyT, HAS_IDX, ITEMS>())) {
        special = special | is_nan_or_negative_zero(raw);
      }
    } else {
#pragma unroll
      for (int n = 0; n < NW; ++n) {
        w[i][n] = 0;
      }
    }
    if constexpr (CARRY) {
      pos2[i / 2] = (i % 2 == 0) ? o : (pos2[i / 2] | (o << 16));
    }
  }
  // float rows without a NaN or a -0.0 (keys-only sorts look for them): the ordered words are
  // then a bijection of the bits
  const bool plain_floats = (CODEC == CODEC_FLOAT) && !HAS_IDX && (__builtin_amdgcn_ballot_w64(special) == 0);
  // passes on whose digit the whole row agrees are the identity permutation: skip them
  uint32_t active = 0;
#pragma unroll
  for (int n = 0; n < NW; ++n) {
    const uint32_t v = wave_all_and(vary_and[n]) ^ wave_all_or(vary_or[n]);
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      if (n * 4 + b < PASSES && ((v >> (8 * b)) & 0xFFu) != 0) {
        active |= 1u << (n * 4 + b);
      }
    }
  }

  // Wide keys: run the passes of the leading varying digits only (2*log2(n) + 4 bits put n keys
  // in order almost always), then check every neighbouring pair on the whole key; pairs out of
  // order are repaired by a few rounds of odd-even transposition, and if that does not finish,
  // all passes run from the state reached (still a stable sort of the input).
  uint32_t todo = active;
  bool shortcut = false;
  // 4-byte keys: worth it for rows of up to 256 elements (2 or 3 leading digits instead of 4)
  constexpr bool SHORTCUT_OK = PASSES >= 5 || (PASSES == 4 && ITEMS <= 4);
  constexpr int MARGIN       = (PASSES == 4) ? 1 : 2;  // passes the shortcut must save to be tried
  if constexpr (SHORTCUT_OK) {
    const int lead = (2 * (32 - __builtin_clz(seg - 1 | 1u)) + 4 + RADIX_BITS - 1) / RADIX_BITS;
    if (__builtin_popcount(active) >= lead + MARGIN) {
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

  // Sorts that return keys only: the first pass to run need not be stable (keys that tie in every
  // digit are the same bits, unless a float row holds a NaN or a -0.0; complex keys are left out),
  // so its ranks come from one LDS atomic per key instead of the ballots of the stable ranking.
  const bool free_first = !HAS_IDX && (OW::BIJECT || plain_floats);
  bool first_running    = true;
  if constexpr (SPLIT_OK) {
    // (with positions: the ranges are steps of the value, which a NaN does not have, so float rows
    // with a NaN, or a -0.0, which the same test reports, keep the passes)
    bool split_ok = free_first;
    if constexpr (HAS_IDX) {
      split_ok = (CODEC != CODEC_FLOAT) || (__builtin_amdgcn_ballot_w64(special) == 0);
    }
    if (split_ok && __builtin_popcount(active) >= 3) {  // uniform for the wave; fewer varying digits: the passes are cheap
      // smallest and largest image of the row (image order is key order)
      uint32_t lo = 0xFFFFFFFFu, hi = 0;
#pragma unroll
      for (int i = 0; i < ITEMS; ++i) {
        if (full || (i * WAVE + lane < seg)) {
          lo = w[i][0] < lo ? w[i][0] : lo;
          hi = w[i][0] > hi ? w[i][0] : hi;
        }
      }
#pragma unroll
      for (int d = 1; d < WAVE; d <<= 1) {
        const uint32_t a = __shfl_xor(lo, d, WAVE), b = __shfl_xor(hi, d, WAVE);
        lo               = a < lo ? a : lo;
        hi               = b > hi ? b : hi;
      }
      // The range of a key.  Integers: the distance of the image from the smallest one, shifted down
      // until the largest distance fits.  Floats: equal steps of the value (the image is stepped in
      // equal ratios, which would crowd the keys of the largest magnitudes); subtraction, scaling
      // and truncation never decrease with the key, so a key in a lower range is a smaller key.
      constexpr int BINS_LOG2 = 31 - __builtin_clz(static_cast<unsigned>(BINS));
      int shift               = 0;
      float origin = 0.0f, scale = 0.0f;
      if constexpr (CODEC == CODEC_FLOAT) {
        const uint32_t lo_bits = sign_unflip(lo), hi_bits = sign_unflip(hi);
        float top;
        __builtin_memcpy(&origin, &lo_bits, 4);
        __builtin_memcpy(&top, &hi_bits, 4);
        scale = static_cast<float>(BINS) / (top - origin);  // (an infinite span gives 0: one crowded range, see bin_of)
      } else {
        const int bits = 32 - __builtin_clz((hi - lo) | 1u);
        shift          = bits > BINS_LOG2 ? bits - BINS_LOG2 : 0;
      }
      auto bin_of = [&](uint32_t image) -> uint32_t {
        if constexpr (CODEC == CODEC_FLOAT) {
          const uint32_t raw = sign_unflip(image);
          float v;
          __builtin_memcpy(&v, &raw, 4);
          // clamped as a float first: the product is NaN or infinite when the row holds an infinity or
          // its span underflows (fmax returns its other operand for a NaN), and converting such a
          // value to an integer is undefined
          const float t = __builtin_fminf(__builtin_fmaxf((v - origin) * scale, 0.0f), static_cast<float>(BINS - 1));
          return static_cast<uint32_t>(t);
        } else {
          return (image - lo) >> shift;
        }
      };
      constexpr int PER_LANE = BINS / WAVE;  // bins a lane scans: a multiple of 4
#pragma unroll
      for (int j = 0; j < PER_LANE / 4; ++j) {
        reinterpret_cast<uint4*>(ctr)[j * WAVE + lane] = make_uint4(0u, 0u, 0u, 0u);
      }
      __builtin_amdgcn_wave_barrier();
      uint32_t bin[ITEMS];
#pragma unroll
      for (int i = 0; i < ITEMS; ++i) {
        bin[i] = bin_of(w[i][0]);
        if (full || (i * WAVE + lane < seg)) {
          atomicAdd(&ctr[bin[i]], 1u);
        }
      }
      __builtin_amdgcn_wave_barrier();
      // exclusive scan: lane l owns bins [l*PER_LANE, (l+1)*PER_LANE)
      uint32_t cnt[PER_LANE], total = 0, largest = 0;
#pragma unroll
      for (int j = 0; j < PER_LANE; ++j) {
        cnt[j] = ctr[lane * PER_LANE + j];
        total += cnt[j];
        largest = cnt[j] > largest ? cnt[j] : largest;
      }
      if (__builtin_amdgcn_ballot_w64(largest > WAVE_SPLIT_LIMIT) == 0) {
        uint32_t run = wave_inclusive_sum_dpp(total) - total;
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int j = 0; j < PER_LANE; ++j) {
          ctr[lane * PER_LANE + j] = run;
          run += cnt[j];
        }
        __builtin_amdgcn_wave_barrier();
        // every key into its range, in whatever order the atomics hand out
        auto pos_of = [&](int i) -> uint32_t { return (pos2[i / 2] >> (16 * (i % 2))) & 0xFFFFu; };
        uint32_t self[HAS_IDX ? 1 : ITEMS];  // where this lane's key i went (without positions: breaks the ties below)
#pragma unroll
        for (int i = 0; i < ITEMS; ++i) {
          if constexpr (!HAS_IDX) {
            self[i] = 0;
          }
          if (full || (i * WAVE + lane < seg)) {
            const uint32_t went    = atomicAdd(&ctr[bin[i]], 1u);
            s_words[wave][0][went] = w[i][0];
            if constexpr (HAS_IDX) {
              s_pos[wave][went] = static_cast<uint16_t>(pos_of(i));
            } else {
              self[i] = went;
            }
          }
        }
        __builtin_amdgcn_wave_barrier();
        // A range now ends where its counter stands and starts where the range before it ends.  A
        // key goes to the start of its range plus the number of keys of the range that come before
        // it: smaller ones, and equal ones that the atomics placed earlier (equal keys are the same
        // bits here; the rule only keeps the places distinct).  All keys of a lane walk in step; a
        // read past the end of a range fetches a key of a later range and is not counted.
        uint32_t from[ITEMS], len[ITEMS], before[ITEMS];
        uint32_t longest = 0;
#pragma unroll
        for (int i = 0; i < ITEMS; ++i) {
          from[i] = 0, len[i] = 0, before[i] = 0;
          if (full || (i * WAVE + lane < seg)) {
            from[i] = (bin[i] == 0) ? 0u : ctr[bin[i] - 1];
            len[i]  = ctr[bin[i]] - from[i];
            if constexpr (!HAS_IDX) {
              self[i] -= from[i];
            }
            longest = len[i] > longest ? len[i] : longest;
          }
        }
        for (uint32_t j = 0; j < longest; ++j) {
          uint32_t other[ITEMS];
          uint32_t other_pos[HAS_IDX ? ITEMS : 1];
#pragma unroll
          for (int i = 0; i < ITEMS; ++i) {
            const uint32_t at = from[i] + j;
            const uint32_t in = at < static_cast<uint32_t>(TILE) ? at : static_cast<uint32_t>(TILE - 1);
            other[i]          = s_words[wave][0][in];
            if constexpr (HAS_IDX) {
              other_pos[i] = s_pos[wave][in];
            }
          }
#pragma unroll
          for (int i = 0; i < ITEMS; ++i) {
            // (bitwise, not short-circuit: no branch between the reads of a round)
            bool first;
            if constexpr (HAS_IDX) {
              first = (other[i] < w[i][0]) | ((other[i] == w[i][0]) & (other_pos[i] < pos_of(i)));
            } else {
              first = (other[i] < w[i][0]) | ((other[i] == w[i][0]) & (j < self[i]));
            }
            before[i] += (first & (j < len[i])) ? 1u : 0u;
          }
        }
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int i = 0; i < ITEMS; ++i) {
          if (full || (i * WAVE + lane < seg)) {
            s_words[wave][0][from[i] + before[i]] = w[i][0];
            if constexpr (HAS_IDX) {
              s_pos[wave][from[i] + before[i]] = static_cast<uint16_t>(pos_of(i));
            }
          }
        }
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int i = 0; i < ITEMS; ++i) {
          if (full || (i * WAVE + lane < seg)) {
            w[i][0] = s_words[wave][0][i * WAVE + lane];
            if constexpr (HAS_IDX) {
              const uint32_t p = s_pos[wave][i * WAVE + lane];
              pos2[i / 2]      = (i % 2 == 0) ? ((pos2[i / 2] & 0xFFFF0000u) | p) : ((pos2[i / 2] & 0xFFFFu) | (p << 16));
            }
          }
        }
        __builtin_amdgcn_wave_barrier();
        todo     = 0;  // sorted: no radix pass is left
        shortcut = false;
      }
    }
  }
  for (;;) {
  for (int pass = 0; pass < PASSES; ++pass) {
    if (((todo >> pass) & 1u) == 0) {
      continue;  // uniform for the wave
    }
    const int word  = pass / 4;
    const int shift = (pass % 4) * 8;
#pragma unroll
    for (int j = 0; j < RADIX / WAVE; ++j) {
      ctr[j * WAVE + lane] = 0;
    }
    __builtin_amdgcn_wave_barrier();
    // ---- rank: counters run from zero ----
    uint32_t dpk[(ITEMS + 3) / 4];   // digits, four per register
    uint32_t rnk2[(ITEMS + 1) / 2];  // ranks, two per register
#pragma unroll
    for (int i = 0; i < ITEMS; ++i) {
      uint32_t wsel = w[i][0];
#pragma unroll
      for (int n = 1; n < NW; ++n) {
        wsel = (word == n) ? w[i][n] : wsel;
      }
      const uint32_t d = (wsel >> shift) & 0xFFu;
      const bool valid = full || (i * WAVE + lane < seg);
      uint32_t r;
      if (!HAS_IDX && free_first && first_running) {  // uniform
        r = valid ? atomicAdd(&ctr[d], 1u) : 0u;
      } else {
        r = wave_match_rank(d, valid, ctr) & 0xFFFFu;
      }
      dpk[i / 4]       = (i % 4 == 0) ? d : (dpk[i / 4] | (d << (8 * (i % 4))));
      rnk2[i / 2]      = (i % 2 == 0) ? r : (rnk2[i / 2] | (r << 16));
      // opaque to the optimiser, which would otherwise keep one register per digit and rank
      asm volatile("" : "+v"(dpk[i / 4]), "+v"(rnk2[i / 2]));
    }
    first_running = false;
    // ---- exclusive scan of the 256 counts: lane l owns digits 4l .. 4l+3 ----
    {
      uint32_t c[RADIX / WAVE], sum = 0;
#pragma unroll
      for (int j = 0; j < RADIX / WAVE; ++j) {
        c[j] = ctr[lane * (RADIX / WAVE) + j];
        sum += c[j];
      }
      uint32_t run = wave_inclusive_scan(sum, lane) - sum;
      __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int j = 0; j < RADIX / WAVE; ++j) {
        ctr[lane * (RADIX / WAVE) + j] = run;
        run += c[j];
      }
    }
    __builtin_amdgcn_wave_barrier();
    // ---- exchange through LDS ----
#pragma unroll
    for (int i = 0; i < ITEMS; ++i) {
      if (full || (i * WAVE + lane < seg)) {
        const uint32_t p = ctr[(dpk[i / 4] >> (8 * (i % 4))) & 0xFFu] + ((rnk2[i / 2] >> (16 * (i % 2))) & 0xFFFFu);
#pragma unroll
        for (int n = 0; n < NW; ++n) {
          s_words[wave][n][p] = w[i][n];
        }
        if constexpr (CARRY) {
          s_pos[wave][p] = static_cast<uint16_t>(pos2[i / 2] >> (16 * (i % 2)));
        }
      }
    }
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int i = 0; i < ITEMS; ++i) {
      const uint32_t o = i * WAVE + lane;
      if (full || o < seg) {
#pragma unroll
        for (int n = 0; n < NW; ++n) {
          w[i][n] = s_words[wave][n][o];
        }
        if constexpr (CARRY) {
          const uint32_t q = s_pos[wave][o];
          pos2[i / 2]      = (i % 2 == 0) ? q : (pos2[i / 2] | (q << 16));
        }
      }
    }
    __builtin_amdgcn_wave_barrier();
  }
    if (!shortcut) {
      break;
    }
    // s_words holds the row as ordered by the leading digits; a few misordered neighbours (keys
    // that tie on those digits) are repaired by rounds of odd-even transposition, which only
    // exchanges strictly misordered pairs and so keeps equal keys in input order
    bool in_order = false;
    for (int round = 0;; ++round) {
      bool bad = false;
#pragma unroll
      for (int i = 0; i < ITEMS; ++i) {
        const uint32_t o = i * WAVE + lane;
        if (o + 1 < seg) {
          bool gt = false, eq = true;  // this key > its right neighbour, most significant word first
#pragma unroll
          for (int n = NW - 1; n >= 0; --n) {
            const uint32_t b = s_words[wave][n][o + 1];
            gt               = gt || (eq && w[i][n] > b);
            eq               = eq && (w[i][n] == b);
          }
          bad = bad || gt;
        }
      }
      if (__builtin_amdgcn_ballot_w64(bad) == 0) {
        in_order = true;
        break;
      }
      if (round == FIXUP_ROUNDS) {
        break;
      }
      __builtin_amdgcn_wave_barrier();
      for (uint32_t phase = 0; phase < 2; ++phase) {
        for (uint32_t q = 2 * lane + phase; q + 1 < seg; q += 2 * WAVE) {
          uint32_t a[NW], b[NW];
          bool gt = false, eq = true;
#pragma unroll
          for (int n = NW - 1; n >= 0; --n) {
            a[n] = s_words[wave][n][q];
            b[n] = s_words[wave][n][q + 1];
            gt   = gt || (eq && a[n] > b[n]);
            eq   = eq && (a[n] == b[n]);
          }
          if (gt) {
#pragma unroll
            for (int n = 0; n < NW; ++n) {
              s_words[wave][n][q]     = b[n];
              s_words[wave][n][q + 1] = a[n];
            }
            if constexpr (CARRY) {
              const uint16_t t   = s_pos[wave][q];
              s_pos[wave][q]     = s_pos[wave][q + 1];
              s_pos[wave][q + 1] = t;
            }
          }
        }
        __builtin_amdgcn_wave_barrier();
      }
#pragma unroll
      for (int i = 0; i < ITEMS; ++i) {
        const uint32_t o = i * WAVE + lane;
        if (full || o < seg) {
#pragma unroll
          for (int n = 0; n < NW; ++n) {
            w[i][n] = s_words[wave][n][o];
          }
          if constexpr (CARRY) {
            const uint32_t q = s_pos[wave][o];
            pos2[i / 2]      = (i % 2 == 0) ? q : (pos2[i / 2] | (q << 16));
          }
        }
      }
      __builtin_amdgcn_wave_barrier();
    }
    if (in_order) {
      break;
    }
    shortcut = false;
    todo     = active;
  }

  // ---- results ----
  if (keys_out != nullptr) {
    if constexpr (FLOAT_KEYS_ONLY) {
      if (!plain_floats) {
        // The zeros of the row (either sign) and its NaNs (any payload) form one block each in the
        // sorted row; a stable sort leaves them there in input order.  Where the blocks start
        // follows from the sorted images.  The images go to LDS; the input is read once more and
        // the bits of every zero and NaN replace the image at their place; then the row is
        // written, decoded outside the two blocks.  All reads of the input come before the first
        // store (keys_out may alias keys_in).  A rare path: plain loops keep its registers few.
        constexpr KeyT SIGN = FloatLayout<KeyT>::sign;
        constexpr KeyT INF  = FloatLayout<KeyT>::inf;
        constexpr KeyT ONES = static_cast<KeyT>(~static_cast<KeyT>(0));
        uint32_t zero_start = 0, zero_end = 0, nan_start = 0;
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int i = 0; i < ITEMS; ++i) {
          const uint32_t o = i * WAVE + lane;
          const bool valid = full || o < seg;
          uint64_t image   = w[i][0];
          if constexpr (NW > 1) {
            image |= static_cast<uint64_t>(w[i][1]) << 32;
          }
          const KeyT img = static_cast<KeyT>(image);
          zero_start += static_cast<uint32_t>(__builtin_popcountll(__builtin_amdgcn_ballot_w64(valid && img < SIGN)));
          zero_end += static_cast<uint32_t>(__builtin_popcountll(__builtin_amdgcn_ballot_w64(valid && img <= SIGN)));
          nan_start += static_cast<uint32_t>(__builtin_popcountll(__builtin_amdgcn_ballot_w64(valid && img != ONES)));
          if (valid) {
#pragma unroll
            for (int n = 0; n < NW; ++n) {
              s_words[wave][n][o] = w[i][n];
            }
          }
        }
        __builtin_amdgcn_wave_barrier();
        auto put = [&](uint32_t slot, KeyT bits) {
          s_words[wave][0][slot] = static_cast<uint32_t>(bits);
          if constexpr (NW > 1) {
            s_words[wave][1][slot] = static_cast<uint32_t>(static_cast<uint64_t>(bits) >> 32);
          }
        };
        uint32_t zeros_seen = 0, nans_seen = 0;
#pragma nounroll
        for (int i = 0; i < ITEMS; ++i) {
          const uint32_t o   = i * WAVE + lane;
          const bool valid   = full || o < seg;
          const KeyT raw     = valid ? keys_in[base + o] : KeyT{};
          const KeyT mag     = static_cast<KeyT>(raw & static_cast<KeyT>(~SIGN));
          const bool is_zero = valid && mag == 0;
          const bool is_nan  = valid && mag > INF;
          const uint64_t bz  = __builtin_amdgcn_ballot_w64(is_zero);
          const uint64_t bn  = __builtin_amdgcn_ballot_w64(is_nan);
          if (is_zero) {
            put(zero_start + zeros_seen + lanes_below(bz), raw);
          }
          if (is_nan) {
            put(nan_start + nans_seen + lanes_below(bn), raw);
          }
          zeros_seen += static_cast<uint32_t>(__builtin_popcountll(bz));
          nans_seen += static_cast<uint32_t>(__builtin_popcountll(bn));
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __builtin_amdgcn_wave_barrier();
#pragma nounroll
        for (int i = 0; i < ITEMS; ++i) {
          const uint32_t o = i * WAVE + lane;
          if (full || o < seg) {
            uint64_t bits = s_words[wave][0][o];
            if constexpr (NW > 1) {
              bits |= static_cast<uint64_t>(s_words[wave][1][o]) << 32;
            }
            const bool in_block = (o >= zero_start && o < zero_end) || o >= nan_start;
            const KeyT value    = static_cast<KeyT>(bits);
            keys_out[base + o]  = in_block ? value : sign_unflip(value);
          }
        }
        return;
      }
    }
    KeyT v[ITEMS];
#pragma unroll
    for (int i = 0; i < ITEMS; ++i) {
      const uint32_t o = i * WAVE + lane;
      if (full || o < seg) {
        if constexpr (OW::BIJECT) {
          v[i] = OW::decode(w[i]);
        } else if constexpr (FLOAT_KEYS_ONLY) {
          v[i] = OW::decode_plain_float(w[i]);  // zeros come out as +0.0, NaNs as some NaN: repaired below
        } else {
          v[i] = keys_in[base + ((pos2[i / 2] >> (16 * (i % 2))) & 0xFFFFu)];  // every gather of the row is issued before any store
        }
      } else {
        v[i] = KeyT{};
      }
    }
    if constexpr (CARRY && !OW::BIJECT) {
      // keys_out may alias keys_in: every gather of the row must have returned before the
      // first store overwrites it (the asm also keeps the compiler from moving either across)
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
#pragma unroll
    for (int i = 0; i < ITEMS; ++i) {
      const uint32_t o = i * WAVE + lane;
      if (full || o < seg) {
        keys_out[base + o] = v[i];
      }
    }
  }
  if constexpr (HAS_IDX) {
#pragma unroll
    for (int i = 0; i < ITEMS; ++i) {
      const uint32_t o = i * WAVE + lane;
      if (full || o < seg) {
        idx_out[base + o] = static_cast<int64_t>((pos2[i / 2] >> (16 * (i % 2))) & 0xFFFFu) + index_offset;
      }
    }
  }
}

}  // namespace cpn
