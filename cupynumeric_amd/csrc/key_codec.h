// Key codecs: map the raw bits of an element to an unsigned integer whose natural order is
// NumPy's sort order for that element type.  Memory always holds raw bits; the mapping is
// applied in registers when a radix digit is extracted, so sorted values keep their exact
// bit patterns (NaN payloads, zero signs) and no decode pass exists.
//
// The reference delegates this to cub's radix traits (src/cupynumeric/sort/cub_sort.cuh:60-182),
// which order floats by bit pattern; the NumPy rule used here differs for NaN and -0.0.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace cpn {

enum Codec : int {
  CODEC_UNSIGNED = 0,  // bool, uint8/16/32/64: identity
  CODEC_SIGNED   = 1,  // int8/16/32/64: flip the sign bit
  CODEC_FLOAT    = 2   // float16/32/64: NaN -> all ones, -0 -> +0, then sign-magnitude flip
};

template <typename U>
struct FloatLayout;
template <>
struct FloatLayout<uint16_t> {
  static constexpr uint16_t sign = 0x8000u;
  static constexpr uint16_t inf  = 0x7C00u;
};
template <>
struct FloatLayout<uint32_t> {
  static constexpr uint32_t sign = 0x80000000u;
  static constexpr uint32_t inf  = 0x7F800000u;
};
template <>
struct FloatLayout<uint64_t> {
  static constexpr uint64_t sign = 0x8000000000000000ull;
  static constexpr uint64_t inf  = 0x7FF0000000000000ull;
};
// 8-bit keys never use the float codec; the specialisation only keeps templates well formed.
template <>
struct FloatLayout<uint8_t> {
  static constexpr uint8_t sign = 0x80u;
  static constexpr uint8_t inf  = 0x78u;
};

// Order-preserving unsigned image of `raw`.
template <int CODEC, typename U>
__host__ __device__ __forceinline__ U ordered_bits(U raw)
{
  if constexpr (CODEC == CODEC_UNSIGNED) {
    return raw;
  } else if constexpr (CODEC == CODEC_SIGNED) {
    return static_cast<U>(raw ^ (static_cast<U>(1) << (sizeof(U) * 8 - 1)));
  } else {
    constexpr U sign = FloatLayout<U>::sign;
    constexpr U inf  = FloatLayout<U>::inf;
    const U mag      = static_cast<U>(raw & static_cast<U>(~sign));
    if (mag > inf) {
      return static_cast<U>(~static_cast<U>(0));  // every NaN ties at the maximum
    }
    if (mag == 0) {
      return sign;  // -0.0 and +0.0 share one key
    }
    return (raw & sign) ? static_cast<U>(~raw) : static_cast<U>(raw | sign);
  }
}

template <int CODEC, typename U>
__host__ __device__ __forceinline__ uint32_t radix_digit(U raw, int shift)
{
  return static_cast<uint32_t>(ordered_bits<CODEC, U>(raw) >> shift) & 0xFFu;
}

}  // namespace cpn
