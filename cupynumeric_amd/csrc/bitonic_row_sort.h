// Short rows of real keys of up to 8 bytes (how long: bitonic_row_limit, 128 ... 1024 keys), sorted by a
// network of compare-exchanges on words held in registers, E = 8 ... 16 elements per lane: element i of a row
// sits in register i % E of the row's lane i / E, a row takes a power of two of lanes (1 ... 64, with the E that
// covers it) and a wavefront holds 64 / lanes rows.  The exchanges between elements of one lane happen between
// its registers, only the others cross lanes, through DPP and swizzle moves: of the 28 steps of a row of 128
// keys on 16 lanes of 8, 18 are inside the lanes and 10 cross them.  (One element per lane, the layout this
// kernel started with, crosses lanes in all 28 steps: 2^26 float32 keys in rows of 128 took 0.28 ms, rows of 32
// 0.25, rows of 8 0.20.)
//
// What is compared: a sort that returns values only, on keys whose image is a bijection of their bits
// (integers; floats when no row of the wavefront holds a NaN or a -0.0), sorts the bare images and maps
// them back (2^26 float32 keys in rows of 128 0.11 ms, of 32 0.09: the speed of the memory).  Otherwise
// the words are (order-preserving image of the key, position in the row) as one word (32 bits for 1- and
// 2-byte keys; for 4-byte keys a double whose mantissa holds both; an image and a position word for 8-byte
// keys), so that no two are equal: the network, which is not stable by itself, then yields exactly the stable order (NaNs tie with each other and +0.0 with -0.0 in the image,
// and the position decides); the raw keys do not travel: they wait in LDS, and every lane fetches the
// keys of the positions that ended up in its slots once, at the end (rows of 128 float32 keys with positions
// out 0.15 ms).  Slots past the end of a row hold the largest image and sort behind, or
// beside, every real element.
//
// Memory is read and written in whole contiguous stretches: a lane of a full row moves its eight
// neighbouring elements as 16-byte vectors; rows that are not full go through LDS, where the rows of
// a wavefront lie as they do in memory, copied in and out with neighbouring lanes on neighbouring
// elements.
//
// Stands, for such rows, where the reference sorts (segment id, value) tuples with a merge sort
// (src/cupynumeric/sort/thrust_sort.cuh:68-122).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "key_codec.h"
#include "radix_common.h"

namespace cpn {

// The value of lane (lane ^ J) of the same wavefront.
template <int J>
__device__ __forceinline__ uint32_t lane_xor(uint32_t v)
{
  static_assert(J == 1 || J == 2 || J == 4 || J == 8 || J == 16 || J == 32, "one bit");
  if constexpr (J == 1) {
    return static_cast<uint32_t>(__builtin_amdgcn_mov_dpp(static_cast<int>(v), 0xB1, 0xF, 0xF, true));  // quad_perm [1,0,3,2]
  } else if constexpr (J == 2) {
    return static_cast<uint32_t>(__builtin_amdgcn_mov_dpp(static_cast<int>(v), 0x4E, 0xF, 0xF, true));  // quad_perm [2,3,0,1]
  } else if constexpr (J == 8) {
    return static_cast<uint32_t>(__builtin_amdgcn_mov_dpp(static_cast<int>(v), 0x128, 0xF, 0xF, true));  // row_ror:8
  } else if constexpr (J == 4 || J == 16) {
    return static_cast<uint32_t>(__builtin_amdgcn_ds_swizzle(static_cast<int>(v), (J << 10) | 0x1F));  // xor mask within 32 lanes
  } else {
    return static_cast<uint32_t>(__shfl_xor(static_cast<int>(v), 32, WAVE));
  }
}
template <int J>
__device__ __forceinline__ uint64_t lane_xor(uint64_t v)
{
  const uint32_t lo = lane_xor<J>(static_cast<uint32_t>(v));
  const uint32_t hi = lane_xor<J>(static_cast<uint32_t>(v >> 32));
  return (static_cast<uint64_t>(hi) << 32) | lo;
}

// 8-byte keys: the image and the position side by side, compared image first.  Two elements per
// lane (rows of 65 ... 128) pay off for them as well once the select between two words is written
// member by member (below): 2^26 float64 keys in rows of 128 0.49 ms through the ranking kernel,
// 0.42 ms here (0.62 ms while the select went through memory).
struct ImagePos {
  uint64_t image;
  uint64_t pos;  // (64 bits so that the struct has no padding; 32 of them travel)
};
template <int J>
__device__ __forceinline__ ImagePos lane_xor(ImagePos v)
{
  return ImagePos{lane_xor<J>(v.image), lane_xor<J>(static_cast<uint32_t>(v.pos))};
}
__device__ __forceinline__ bool operator<(const ImagePos& a, const ImagePos& b)
{
  return a.image < b.image || (a.image == b.image && static_cast<uint32_t>(a.pos) < static_cast<uint32_t>(b.pos));
}
// (member by member: a select between two structs goes through their addresses, i.e. through memory)
__device__ __forceinline__ ImagePos word_select(bool first, const ImagePos& a, const ImagePos& b)
{
  return ImagePos{first ? a.image : b.image, first ? a.pos : b.pos};
}
__device__ __forceinline__ uint32_t word_select(bool first, uint32_t a, uint32_t b) { return first ? a : b; }
__device__ __forceinline__ uint64_t word_select(bool first, uint64_t a, uint64_t b) { return first ? a : b; }
__device__ __forceinline__ uint32_t word_pos(uint32_t w) { return w; }
__device__ __forceinline__ uint32_t word_pos(uint64_t w) { return static_cast<uint32_t>(w); }
__device__ __forceinline__ uint32_t word_pos(const ImagePos& w) { return static_cast<uint32_t>(w.pos); }

// A float64 key compared as the number it is (rows without NaN and -0.0 only, where that is the order of
// the images): the exchange inside a lane is a min and a max instruction instead of a 64-bit integer
// compare and four selects.
struct F64Word {
  double v;
};
template <int J>
__device__ __forceinline__ F64Word lane_xor(F64Word w)
{
  return F64Word{__longlong_as_double(static_cast<long long>(lane_xor<J>(static_cast<uint64_t>(__double_as_longlong(w.v)))))};
}
__device__ __forceinline__ F64Word word_select(bool first, const F64Word& a, const F64Word& b) { return F64Word{first ? a.v : b.v}; }
// (image of a 4-byte key, position in the row) as a number: the 52 bits image << 20 | position are the
// mantissa of a double of the fixed exponent 2^52, so the numbers order as the pairs do and are all finite.
__device__ __forceinline__ F64Word pack_image_pos(uint32_t image, uint32_t pos)
{
  const uint64_t bits = 0x4330000000000000ull | (static_cast<uint64_t>(image) << 20) | pos;
  return F64Word{__longlong_as_double(static_cast<long long>(bits))};
}
__device__ __forceinline__ uint32_t word_pos(const F64Word& w) { return static_cast<uint32_t>(__double_as_longlong(w.v)) & 0xFFFFFu; }

// Elements per lane: eight for full rows (ten, twelve or fourteen for rows in between, see the network below), or
// sixteen where a sort returns values only of full rows of 8-byte keys (fewer of the steps cross lanes: 6
// instead of 10 of the 28 steps of a row of 128 keys.  2^26 float64 keys in rows of 32 0.29 -> 0.19 ms, of 128
// 0.31 -> 0.23; int64 0.21 and 0.27.  Plain sorts of 4-byte keys, which already move at the speed of the
// memory with eight, lose to the hand-over in LDS that sixteen need: rows of 128 float32 keys 0.11 -> 0.14 ms.)
constexpr int BLOCKED_E = 8;

// a < b on the words of the network.  (For 64-bit words the borrow of a subtraction and a compare of the
// halves were measured against the plain compare: the same and 10 % slower on rows of 128 keys.)
__device__ __forceinline__ bool word_less(uint32_t a, uint32_t b) { return a < b; }
__device__ __forceinline__ bool word_less(uint64_t a, uint64_t b) { return a < b; }
__device__ __forceinline__ bool word_less(const ImagePos& a, const ImagePos& b) { return a < b; }
__device__ __forceinline__ bool word_less(const F64Word& a, const F64Word& b) { return a.v < b.v; }

// The value of lane (lane ^ M) for M = 2^k - 1: the lane's mirror image inside its group of M + 1 lanes.
template <int M>
__device__ __forceinline__ uint32_t lane_mirror(uint32_t v)
{
  static_assert(M == 1 || M == 3 || M == 7 || M == 15 || M == 31 || M == 63, "all bits below a power of two");
  if constexpr (M == 1) {
    return static_cast<uint32_t>(__builtin_amdgcn_mov_dpp(static_cast<int>(v), 0xB1, 0xF, 0xF, true));  // quad_perm [1,0,3,2]
  } else if constexpr (M == 3) {
    return static_cast<uint32_t>(__builtin_amdgcn_mov_dpp(static_cast<int>(v), 0x1B, 0xF, 0xF, true));  // quad_perm [3,2,1,0]
  } else if constexpr (M == 7) {
    return static_cast<uint32_t>(__builtin_amdgcn_mov_dpp(static_cast<int>(v), 0x141, 0xF, 0xF, true));  // row_half_mirror
  } else if constexpr (M == 15) {
    return static_cast<uint32_t>(__builtin_amdgcn_mov_dpp(static_cast<int>(v), 0x140, 0xF, 0xF, true));  // row_mirror
  } else if constexpr (M == 31) {
    return static_cast<uint32_t>(__builtin_amdgcn_ds_swizzle(static_cast<int>(v), (0x1F << 10) | 0x1F));  // xor mask within 32 lanes
  } else {
    return static_cast<uint32_t>(__shfl_xor(static_cast<int>(v), 63, WAVE));
  }
}
template <int M>
__device__ __forceinline__ uint64_t lane_mirror(uint64_t v)
{
  const uint32_t lo = lane_mirror<M>(static_cast<uint32_t>(v));
  const uint32_t hi = lane_mirror<M>(static_cast<uint32_t>(v >> 32));
  return (static_cast<uint64_t>(hi) << 32) | lo;
}
template <int M>
__device__ __forceinline__ ImagePos lane_mirror(ImagePos v)
{
  return ImagePos{lane_mirror<M>(v.image), lane_mirror<M>(static_cast<uint32_t>(v.pos))};
}
template <int M>
__device__ __forceinline__ F64Word lane_mirror(F64Word w)
{
  return F64Word{__longlong_as_double(static_cast<long long>(lane_mirror<M>(static_cast<uint64_t>(__double_as_longlong(w.v)))))};
}

// One compare-exchange between two registers of a lane: the smaller word goes to `lo`.
template <typename W>
__device__ __forceinline__ void blocked_exchange_in_lane(W& lo, W& hi)
{
  const W a = lo, b = hi;
  if constexpr (std::is_same_v<W, uint32_t>) {
    lo = a < b ? a : b;  // (one min and one max instruction)
    hi = a < b ? b : a;
  } else if constexpr (std::is_same_v<W, F64Word>) {
    // (written out: the compiler's fmin / fmax put an instruction in front of each operand that quiets
    // signalling NaNs, which these rows do not hold)
    asm("v_min_f64 %0, %1, %2" : "=v"(lo.v) : "v"(a.v), "v"(b.v));
    asm("v_max_f64 %0, %1, %2" : "=v"(hi.v) : "v"(a.v), "v"(b.v));
  } else {
    const bool swap = word_less(b, a);
    lo              = word_select(swap, b, a);
    hi              = word_select(swap, a, b);
  }
}

// The network.  A lane first sorts its own E elements; then, level by level, the sorted runs of 1, 2, 4 ...
// lanes are merged in pairs: a merge starts by comparing every element with its mirror image in the run of
// both (register E - 1 - r of the mirrored lane), goes on with the same register of the lanes at distance
// KL / 4 ... 1, and ends inside the lanes, whose elements are a bitonic sequence by then.  The smaller word
// always goes to the smaller element number, so no step has to know which way its run points.  E need not be
// a power of two: a row of n keys takes 1, 2, 4 ... 32 lanes of 8, 10, 12, 14 or 16 elements each, whichever
// covers it, instead of the next power of two of slots.  Inside a lane: Batcher's odd-even merge sort for 16
// elements without the exchanges that touch elements past E (they would compare with padding that is never
// smaller), 19, 32, 42, 53 and 63 exchanges for E = 8 ... 16; a bitonic sequence of an even number of elements
// takes a half-cleaner and becomes two bitonic sequences of half the length, and one of 3, 5 or 7 elements is
// sorted by the smallest known network (3, 9, 16 exchanges).  `sub` is the lane's number inside its row.
template <int A, int B, typename W, int E>
__device__ __forceinline__ void lane_exchange(W (&w)[E])
{
  static_assert(A < B && B < E, "the smaller word goes to the smaller element number");
  blocked_exchange_in_lane(w[A], w[B]);
}
template <int LO, int N, int R, typename W, int E>
__device__ __forceinline__ void oddeven_merge(W (&w)[E])
{
  if constexpr (LO + R < E) {
    constexpr int M = 2 * R;
    if constexpr (M < N) {
      oddeven_merge<LO, N, M>(w);
      oddeven_merge<LO + R, N, M>(w);
#pragma unroll
      for (int i = LO + R; i + R < LO + N; i += M) {
        if (i + R < E) {
          blocked_exchange_in_lane(w[i], w[i + R]);
        }
      }
    } else {
      blocked_exchange_in_lane(w[LO], w[LO + R]);
    }
  }
}
template <int LO, int N, typename W, int E>
__device__ __forceinline__ void oddeven_merge_sort(W (&w)[E])
{
  if constexpr (N > 1 && LO + 1 < E) {
    oddeven_merge_sort<LO, N / 2>(w);
    oddeven_merge_sort<LO + N / 2, N / 2>(w);
    oddeven_merge<LO, N, 1>(w);
  }
}
// Sorts the E elements of a lane, whatever their order.
template <typename W, int E>
__device__ __forceinline__ void lane_sort(W (&w)[E])
{
  static_assert(E > 4 && E <= 16, "elements per lane");
  oddeven_merge_sort<0, (E <= 8 ? 8 : 16)>(w);
}
// Sorts elements OFF ... OFF + M - 1 of a lane, M = 3, 5, 7.
template <int OFF, int M, typename W, int E>
__device__ __forceinline__ void lane_sort_part(W (&w)[E])
{
  if constexpr (M == 3) {
    lane_exchange<OFF + 0, OFF + 2>(w), lane_exchange<OFF + 0, OFF + 1>(w), lane_exchange<OFF + 1, OFF + 2>(w);
  } else if constexpr (M == 5) {
    lane_exchange<OFF + 0, OFF + 3>(w), lane_exchange<OFF + 1, OFF + 4>(w);
    lane_exchange<OFF + 0, OFF + 2>(w), lane_exchange<OFF + 1, OFF + 3>(w);
    lane_exchange<OFF + 0, OFF + 1>(w), lane_exchange<OFF + 2, OFF + 4>(w);
    lane_exchange<OFF + 1, OFF + 2>(w), lane_exchange<OFF + 3, OFF + 4>(w);
    lane_exchange<OFF + 2, OFF + 3>(w);
  } else {
    static_assert(M == 7, "networks for 3, 5 and 7 elements");
    lane_exchange<OFF + 0, OFF + 6>(w), lane_exchange<OFF + 2, OFF + 3>(w), lane_exchange<OFF + 4, OFF + 5>(w);
    lane_exchange<OFF + 0, OFF + 2>(w), lane_exchange<OFF + 1, OFF + 4>(w), lane_exchange<OFF + 3, OFF + 6>(w);
    lane_exchange<OFF + 0, OFF + 1>(w), lane_exchange<OFF + 2, OFF + 5>(w), lane_exchange<OFF + 3, OFF + 4>(w);
    lane_exchange<OFF + 1, OFF + 2>(w), lane_exchange<OFF + 4, OFF + 6>(w);
    lane_exchange<OFF + 2, OFF + 3>(w), lane_exchange<OFF + 4, OFF + 5>(w);
    lane_exchange<OFF + 1, OFF + 2>(w), lane_exchange<OFF + 3, OFF + 4>(w), lane_exchange<OFF + 5, OFF + 6>(w);
  }
}
// Sorts elements OFF ... OFF + M - 1 of a lane, which form a bitonic sequence.
template <int OFF, int M, typename W, int E>
__device__ __forceinline__ void lane_sort_bitonic_part(W (&w)[E])
{
  if constexpr (M > 1) {
    if constexpr (M % 2 == 0) {
#pragma unroll
      for (int i = 0; i < M / 2; ++i) {
        blocked_exchange_in_lane(w[OFF + i], w[OFF + i + M / 2]);
      }
      lane_sort_bitonic_part<OFF, M / 2>(w);
      lane_sort_bitonic_part<OFF + M / 2, M / 2>(w);
    } else {
      lane_sort_part<OFF, M>(w);
    }
  }
}
template <typename W, int E>
__device__ __forceinline__ void lane_sort_bitonic(W (&w)[E])
{
  lane_sort_bitonic_part<0, E>(w);
}
// The steps of a merge that cross lanes: the mirror image in the run of KL lanes, then the lanes at distance D.
template <int KL, typename W, int E>
__device__ __forceinline__ void cross_mirror(W (&w)[E], uint32_t sub)
{
  const bool keep_min = (sub & (KL / 2)) == 0;  // the lower half of the run keeps the smaller words
  W other[E];
#pragma unroll
  for (int r = 0; r < E; ++r) {
    other[r] = lane_mirror<KL - 1>(w[E - 1 - r]);
  }
#pragma unroll
  for (int r = 0; r < E; ++r) {
    w[r] = word_select(word_less(w[r], other[r]) == keep_min, w[r], other[r]);
  }
}
template <int D, typename W, int E>
__device__ __forceinline__ void cross_steps(W (&w)[E], uint32_t sub)
{
  if constexpr (D >= 1) {
    const bool keep_min = (sub & D) == 0;
#pragma unroll
    for (int r = 0; r < E; ++r) {
      const W other = lane_xor<D>(w[r]);
      w[r]          = word_select(word_less(w[r], other) == keep_min, w[r], other);
    }
    cross_steps<D / 2>(w, sub);
  }
}
template <int KL, int LANES, typename W, int E>
__device__ __forceinline__ void merge_levels(W (&w)[E], uint32_t sub)
{
  if constexpr (KL <= LANES) {
    cross_mirror<KL>(w, sub);
    cross_steps<KL / 4>(w, sub);
    lane_sort_bitonic(w);
    merge_levels<2 * KL, LANES>(w, sub);
  }
}
// A row of LANES x E slots.
template <int LANES, typename W, int E>
__device__ __forceinline__ void blocked_sort(W (&w)[E], uint32_t sub)
{
  lane_sort(w);
  merge_levels<2, LANES>(w, sub);
}

// LANES = lanes per row (a power of two), E = elements per lane: LANES x E slots per row (>= row length),
// 64 / LANES rows per wavefront, four wavefronts per workgroup.
template <typename KeyT, int CODEC, bool HAS_IDX, int LANES, int E>
__global__ __launch_bounds__(256) void bitonic_row_sort_kernel(const KeyT* __restrict__ keys_in,
                                                                        KeyT* keys_out,
                                                                        int64_t* __restrict__ idx_out,
                                                                        uint32_t seg,
                                                                        uint64_t rows,
                                                                        int64_t index_offset,
                                                                        uint32_t* status)
{
  static_assert(sizeof(KeyT) <= 8 && (CODEC == CODEC_UNSIGNED || CODEC == CODEC_SIGNED || CODEC == CODEC_FLOAT),
                "real keys of up to 8 bytes");
  static_assert(E >= 8 && E <= 16 && E % 2 == 0, "elements per lane");
  static_assert(LANES >= 1 && LANES <= WAVE && (LANES & (LANES - 1)) == 0, "lanes per row: a power of two");
  constexpr int N = LANES * E;  // slots per row
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    *status = 0;  // the workspace's status word: a per-row sort cannot fail on the device
  }
  // 4-byte keys: image in the high word, position in the low one; shorter keys: image << 16 | position;
  // 8-byte keys: two registers for the image, one for the position
  using W = std::conditional_t<sizeof(KeyT) == 8, ImagePos, std::conditional_t<sizeof(KeyT) == 4, F64Word, uint32_t>>;
  constexpr int ROWS_WAVE = WAVE / LANES;
  constexpr int WAVES     = 256 / WAVE;
  // The stretch of a wavefront in LDS, as it lies in memory.  (A word of padding after every 32, so that lanes
  // whose elements start 8 elements apart do not meet in four banks, was measured and changed nothing: what the
  // rows that go through here pay for is instructions, 94 per key against 68 for rows moved as vectors before
  // the addresses below were made uniform.)
  constexpr int WAVE_SLOTS = WAVE * E;
  __shared__ __align__(16) KeyT s_raw[(256 / WAVE) * WAVE_SLOTS];
  __shared__ __align__(16) uint16_t s_from[HAS_IDX ? 256 * E : 8];

  const uint32_t lane   = threadIdx.x & (WAVE - 1);
  // (the number of the wavefront, read from its first lane so that the compiler knows that everything derived
  // from it is the same in all lanes: the addresses of the stretch then need no vector arithmetic)
  const uint32_t wslot  = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x / WAVE)));
  const uint64_t wave   = static_cast<uint64_t>(blockIdx.x) * WAVES + wslot;
  const uint32_t sub    = lane & (LANES - 1);
  const uint32_t wrow   = lane / LANES;  // row of this lane inside its wavefront
  const uint64_t row    = wave * ROWS_WAVE + wrow;
  const uint64_t base   = row * seg;
  const uint32_t first  = sub * E;  // position of this lane's first element in its row
  const bool row_exists = row < rows;
  const uint32_t row_len = row_exists ? seg : 0u;  // slots of this lane's row that hold keys

  // Full rows whose lanes' eight elements can be moved as 16-byte (single bytes: 8-byte) vectors: a wavefront
  // then reads and writes whole contiguous kilobytes per instruction.  Other rows go through LDS: the rows of
  // a wavefront are one contiguous stretch of memory, which its lanes copy in and out element by element,
  // neighbouring lanes on neighbouring elements, and from which every lane takes the eight elements it owns.
  constexpr int LANE_BYTES = E * static_cast<int>(sizeof(KeyT));
  constexpr bool CAN_VEC   = E == 8 || E == 16;  // (other lanes own a number of bytes that is no whole vector)
  using VecT               = std::conditional_t<(LANE_BYTES >= 16), uint4, uint2>;
  constexpr int VECS       = CAN_VEC ? LANE_BYTES / static_cast<int>(sizeof(VecT)) : 1;
  const bool vec_keys = CAN_VEC && (seg == N) && ((reinterpret_cast<uintptr_t>(keys_in) | reinterpret_cast<uintptr_t>(keys_out)) &
                                       (sizeof(VecT) - 1)) == 0;  // uniform
  const bool vec_idx  = CAN_VEC && (seg == N) && (reinterpret_cast<uintptr_t>(idx_out) & 15u) == 0;
  // the stretch of this wavefront: its rows, densely, as in memory
  const uint64_t wave_row0 = wave * ROWS_WAVE;
  const uint32_t wave_rows =
    wave_row0 >= rows ? 0u : static_cast<uint32_t>(rows - wave_row0 < ROWS_WAVE ? rows - wave_row0 : ROWS_WAVE);
  const uint32_t stretch_len  = wave_rows * seg;  // at most 512 elements
  const uint64_t stretch_base = wave_row0 * seg;
  KeyT* const s_wave          = s_raw + wslot * WAVE_SLOTS;
  KeyT* const dst_keys        = keys_out + stretch_base;  // (used where keys_out is not null)
  const uint32_t row_at       = wrow * seg;  // this lane's row inside the stretch

  // Lanes that own 64 bytes or more (8-byte keys; sixteen elements) and fetched them straight from memory would
  // touch a cache line of their own with every instruction (measured with 64 bytes of float32 keys per lane:
  // rows of 32 keys 0.135 ms against 0.09 with 32 bytes).  So the wavefront moves its stretch in 16-byte
  // pieces, neighbouring lanes on neighbouring pieces, and the pieces change hands in LDS: piece q lies at
  // q ^ ((q >> 3) & 7), which keeps eight neighbouring pieces, and the pieces that eight neighbouring lanes
  // own, in different banks.
  constexpr bool VIA_LDS      = CAN_VEC && LANE_BYTES >= 64;
  constexpr int PIECE_KEYS    = 16 / static_cast<int>(sizeof(KeyT));
  constexpr int PIECES        = VIA_LDS ? LANE_BYTES / 16 : 1;  // per lane
  uint4* const s_pieces       = reinterpret_cast<uint4*>(s_wave);
  const uint32_t stretch_pieces = stretch_len / PIECE_KEYS;
  auto piece_slot = [](uint32_t q) { return q ^ ((q >> 3) & 7u); };
  auto load_full_rows = [&](KeyT (&dst)[E]) {
    if constexpr (!CAN_VEC) {
      (void)dst;
    } else if constexpr (VIA_LDS) {
      const uint4* src = reinterpret_cast<const uint4*>(keys_in + stretch_base);
      uint4 got[PIECES];
#pragma unroll
      for (int k = 0; k < PIECES; ++k) {
        const uint32_t q = k * WAVE + lane;
        got[k]           = uint4{};
        if (q < stretch_pieces) {
          got[k] = src[q];
        }
      }
#pragma unroll
      for (int k = 0; k < PIECES; ++k) {
        s_pieces[piece_slot(k * WAVE + lane)] = got[k];
      }
      __builtin_amdgcn_wave_barrier();  // (a stretch belongs to one wavefront, whose LDS operations execute in order)
      uint4 own[PIECES];
#pragma unroll
      for (int j = 0; j < PIECES; ++j) {
        own[j] = s_pieces[piece_slot(lane * PIECES + j)];
      }
      __builtin_memcpy(dst, own, LANE_BYTES);
    } else {
      VecT q[VECS];
#pragma unroll
      for (int v = 0; v < VECS; ++v) {
        q[v] = VecT{};
        if (row_exists) {
          q[v] = reinterpret_cast<const VecT*>(keys_in + base + first)[v];
        }
      }
      __builtin_memcpy(dst, q, LANE_BYTES);
    }
  };
  auto store_full_rows = [&](const KeyT (&src)[E]) {
    if constexpr (!CAN_VEC) {
      (void)src;
    } else if constexpr (VIA_LDS) {
      uint4 own[PIECES];
      __builtin_memcpy(own, src, LANE_BYTES);
#pragma unroll
      for (int j = 0; j < PIECES; ++j) {
        s_pieces[piece_slot(lane * PIECES + j)] = own[j];
      }
      __builtin_amdgcn_wave_barrier();
      uint4* dst = reinterpret_cast<uint4*>(keys_out + stretch_base);
#pragma unroll
      for (int k = 0; k < PIECES; ++k) {
        const uint32_t q = k * WAVE + lane;
        if (q < stretch_pieces) {
          dst[q] = s_pieces[piece_slot(q)];
        }
      }
    } else {
      if (row_exists) {
        VecT q[VECS];
        __builtin_memcpy(q, src, LANE_BYTES);
#pragma unroll
        for (int v = 0; v < VECS; ++v) {
          reinterpret_cast<VecT*>(keys_out + base + first)[v] = q[v];
        }
      }
    }
  };

  KeyT raw[E];
  if (vec_keys) {
    load_full_rows(raw);
  } else {
    KeyT got[E];
    const KeyT* const src = keys_in + stretch_base;
#pragma unroll
    for (int k = 0; k < E; ++k) {  // (all loads first)
      const uint32_t e = lane + k * WAVE;
      got[k]           = KeyT{};
      if (e < stretch_len) {
        got[k] = src[e];
      }
    }
#pragma unroll
    for (int k = 0; k < E; ++k) {
      s_wave[lane + k * WAVE] = got[k];  // (past the end of the stretch: zeros, which nothing uses)
    }
    __builtin_amdgcn_wave_barrier();  // (a stretch belongs to one wavefront, whose LDS operations execute in order)
    // (a lane reads its E slots whether its row fills them or not: they lie inside the wavefront's part of
    // the array, and what lies past the end of a row is replaced below)
    const KeyT* const own = s_wave + row_at + first;
#pragma unroll
    for (int r = 0; r < E; ++r) {
      raw[r] = own[r];
    }
  }
  // A sort that returns values only, on keys whose image is a bijection of their bits (integers; floats when
  // no row of the wavefront holds a NaN or a -0.0), sorts the bare images, one word per element, and maps
  // them back: equal images are equal keys, so nothing has to tell them apart.
  if constexpr (!HAS_IDX) {
    bool bare = true;  // uniform over the wavefront
    if constexpr (CODEC == CODEC_FLOAT) {
      bool special = false;
#pragma unroll
      for (int r = 0; r < E; ++r) {
        special |= first + r < row_len && is_nan_or_negative_zero(raw[r]);
      }
      bare = __ballot(special) == 0;
    }
    if (bare) {
      constexpr bool NATIVE = CODEC == CODEC_FLOAT && sizeof(KeyT) == 8;  // float64 keys as numbers
      using B = std::conditional_t<NATIVE, F64Word, std::conditional_t<sizeof(KeyT) == 8, uint64_t, uint32_t>>;
      B b[E];
#pragma unroll
      for (int r = 0; r < E; ++r) {
        const bool valid = first + r < row_len;
        // (slots past the end: behind or beside the largest key)
        if constexpr (NATIVE) {
          b[r] = F64Word{valid ? __longlong_as_double(static_cast<long long>(raw[r])) : __builtin_huge_val()};
        } else {
          KeyT image;
          if constexpr (CODEC == CODEC_FLOAT) {
            image = sign_flip<KeyT>(raw[r]);
          } else {
            image = ordered_bits<CODEC, KeyT>(raw[r]);
          }
          b[r] = valid ? static_cast<B>(image) : static_cast<B>(~B{0});
        }
      }
      blocked_sort<LANES>(b, sub);
      KeyT bits[E];
#pragma unroll
      for (int r = 0; r < E; ++r) {
        if constexpr (NATIVE) {
          bits[r] = static_cast<KeyT>(__double_as_longlong(b[r].v));
        } else {
          const KeyT image = static_cast<KeyT>(b[r]);
          if constexpr (CODEC == CODEC_FLOAT) {
            bits[r] = sign_unflip<KeyT>(image);
          } else {
            bits[r] = ordered_bits<CODEC, KeyT>(image);  // (the identity, or the sign bit flipped back)
          }
        }
      }
      if (keys_out == nullptr) {
        return;
      }
      if (vec_keys) {
        store_full_rows(bits);
      } else {
#pragma unroll
        for (int r = 0; r < E; ++r) {
          const uint32_t pos = first + r;
          if (pos < row_len) {
            s_wave[row_at + pos] = bits[r];  // (every lane has read its elements of the stretch; LDS operations of a wavefront execute in order)
          }
        }
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int k = 0; k < E; ++k) {
          const uint32_t e = lane + k * WAVE;
          if (e < stretch_len) {
            dst_keys[e] = s_wave[e];
          }
        }
      }
      return;
    }
  }
  W w[E];
#pragma unroll
  for (int r = 0; r < E; ++r) {
    const uint32_t pos = first + r;
    const bool valid   = pos < row_len;
    // (slots past the end of a row: the largest image, and a position behind every element's)
    const KeyT image = valid ? ordered_bits<CODEC, KeyT>(raw[r]) : static_cast<KeyT>(~KeyT{0});
    if constexpr (sizeof(KeyT) == 8) {
      w[r] = ImagePos{image, pos};
    } else {
      if constexpr (sizeof(KeyT) == 4) {
        w[r] = pack_image_pos(image, pos);
      } else {
        w[r] = (static_cast<W>(image) << 16) | pos;
      }
    }
  }
  blocked_sort<LANES>(w, sub);

  // ---- slot p of the sorted row holds the element that came from position `from` ----
  uint32_t from[E];
#pragma unroll
  for (int r = 0; r < E; ++r) {
    from[r] = word_pos(w[r]) & 0xFFFFu;
  }
  if (keys_out != nullptr) {
    if (vec_keys) {
      // every lane parks its raw keys and takes those of the positions that ended up in its slots
      const uint32_t mine = wrow * N;
#pragma unroll
      for (int r = 0; r < E; ++r) {
        s_wave[mine + first + r] = raw[r];
      }
      __builtin_amdgcn_wave_barrier();
      KeyT bits[E];
#pragma unroll
      for (int r = 0; r < E; ++r) {
        bits[r] = s_wave[mine + from[r]];
      }
      __builtin_amdgcn_wave_barrier();  // (the parked keys have been read before the pieces of the result go to LDS)
      store_full_rows(bits);
    } else {
      // the stretch still holds the raw keys: permute it in place (all reads, then all writes), copy it out
      KeyT bits[E];
#pragma unroll
      for (int r = 0; r < E; ++r) {
        const uint32_t pos = first + r;
        bits[r]            = (pos < row_len) ? s_wave[row_at + from[r]] : KeyT{};
      }
      __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int r = 0; r < E; ++r) {
        const uint32_t pos = first + r;
        if (pos < row_len) {
          s_wave[row_at + pos] = bits[r];
        }
      }
      __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int k = 0; k < E; ++k) {
        const uint32_t e = lane + k * WAVE;
        if (e < stretch_len) {
          dst_keys[e] = s_wave[e];
        }
      }
    }
  }
  if constexpr (HAS_IDX) {
    bool stored = false;
    if constexpr (CAN_VEC) {
     if (vec_idx) {
      stored = true;
      // The positions change hands in LDS as 16-bit words, so that a lane stores two neighbouring int64 words
      // and its neighbours the next ones: a lane that stored the 64 bytes of its own eight slots would touch
      // a cache line of its own with every instruction (2^21 rows of 128 float32 keys: 0.79 ms that way).
      uint16_t* const s_fwave = s_from + wslot * (WAVE * E);
      uint16_t mine[E];
#pragma unroll
      for (int r = 0; r < E; ++r) {
        mine[r] = static_cast<uint16_t>(from[r]);
      }
      uint4 packed[E / 8];
      __builtin_memcpy(packed, mine, sizeof(mine));
#pragma unroll
      for (int v = 0; v < E / 8; ++v) {
        reinterpret_cast<uint4*>(s_fwave)[lane * (E / 8) + v] = packed[v];
      }
      __builtin_amdgcn_wave_barrier();
      uint4* const dst = reinterpret_cast<uint4*>(idx_out + stretch_base);
#pragma unroll
      for (int k = 0; k < E / 2; ++k) {
        const uint32_t q = k * WAVE + lane;  // slots 2 q and 2 q + 1 of the stretch
        if (2 * q < stretch_len) {
          const uint32_t pair = reinterpret_cast<const uint32_t*>(s_fwave)[q];
          const int64_t out[2] = {static_cast<int64_t>(pair & 0xFFFFu) + index_offset,
                                  static_cast<int64_t>(pair >> 16) + index_offset};
          uint4 word;
          __builtin_memcpy(&word, out, sizeof(word));
          dst[q] = word;
        }
      }
     }
    }
    if (!stored) {
      // positions through LDS as well, so that neighbouring lanes store neighbouring int64 words
      uint16_t* const s_fwave = s_from + wslot * (WAVE * E);
      int64_t* const dst_idx  = idx_out + stretch_base;
#pragma unroll
      for (int r = 0; r < E; ++r) {
        const uint32_t pos = first + r;
        if (pos < row_len) {
          s_fwave[wrow * seg + pos] = static_cast<uint16_t>(from[r]);
        }
      }
      __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int k = 0; k < E; ++k) {
        const uint32_t e = lane + k * WAVE;
        if (e < stretch_len) {
          dst_idx[e] = static_cast<int64_t>(s_fwave[e]) + index_offset;
        }
      }
    }
  }
}

}  // namespace cpn
