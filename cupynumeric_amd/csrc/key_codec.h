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
  CODEC_FLOAT    = 2,  // float16/32/64: NaN -> all ones, -0 -> +0, then sign-magnitude flip
  CODEC_COMPLEX  = 3   // complex64/128: (class, primary, secondary) of two float keys, see KeyTraits
};

// Raw bits of a complex128 element: real part in `lo`, imaginary part in `hi`.
struct alignas(16) U128 {
  uint64_t lo;
  uint64_t hi;
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

// The float image without the NaN and zero rules, and its inverse: a bijection of the bits that
// agrees with ordered_bits<CODEC_FLOAT> on every value except NaNs and -0.0.
template <typename U>
__host__ __device__ __forceinline__ U sign_flip(U raw)
{
  constexpr U sign = FloatLayout<U>::sign;
  return (raw & sign) ? static_cast<U>(~raw) : static_cast<U>(raw | sign);
}
template <typename U>
__host__ __device__ __forceinline__ U sign_unflip(U image)
{
  constexpr U sign = FloatLayout<U>::sign;
  return (image & sign) ? static_cast<U>(image ^ sign) : static_cast<U>(~image);
}

// Is the float with these bits a NaN or -0.0: the two kinds of key whose image is shared with keys
// of other bits.  One class-test instruction for 4- and 8-byte floats.
template <typename U>
__device__ __forceinline__ bool is_nan_or_negative_zero(U raw)
{
  constexpr int CLASS_SNAN = 1, CLASS_QNAN = 2, CLASS_NEG_ZERO = 32;  // bits of the class mask
  if constexpr (sizeof(U) == 4) {
    float v;
    __builtin_memcpy(&v, &raw, 4);
    return __builtin_amdgcn_classf(v, CLASS_SNAN | CLASS_QNAN | CLASS_NEG_ZERO);
  } else if constexpr (sizeof(U) == 8) {
    double v;
    __builtin_memcpy(&v, &raw, 8);
    return __builtin_amdgcn_class(v, CLASS_SNAN | CLASS_QNAN | CLASS_NEG_ZERO);
  } else {
    constexpr U sign = FloatLayout<U>::sign;
    return static_cast<U>(raw & static_cast<U>(~sign)) > FloatLayout<U>::inf || raw == sign;
  }
}

template <int CODEC, typename U>
__host__ __device__ __forceinline__ uint32_t radix_digit(U raw, int shift)
{
  return static_cast<uint32_t>(ordered_bits<CODEC, U>(raw) >> shift) & 0xFFu;
}

// What the sort kernels need to know about a key type: how many 8-bit passes sort it, the
// digit of a pass, and the key as 64-bit words whose bytes are those digits (word p/8, byte
// p%8), from which a row finds the passes on which all its keys agree.
template <int CODEC, typename U>
struct KeyTraits {
  static constexpr int PASSES = sizeof(U);
  static constexpr int NWORDS = 1;
  static __host__ __device__ __forceinline__ uint32_t digit(U raw, int pass)
  {
    return radix_digit<CODEC, U>(raw, pass * 8);
  }
  static __host__ __device__ __forceinline__ void words(U raw, uint64_t (&w)[NWORDS])
  {
    w[0] = static_cast<uint64_t>(ordered_bits<CODEC, U>(raw));
  }
};

// NumPy orders complex numbers by (real, imag) with NaNs last in this sense
// (numpy/_core/src/npysort/npysort_common.h, CFLOAT_LT): first every element without NaN,
// by real then imaginary part; then those whose imaginary part only is NaN, by real part;
// then those whose real part is NaN, by imaginary part; last those with two NaNs.  As a radix
// key: class (0..3) most significant, then a primary and a secondary float key
//   class 0: (real, imag)   class 1: (real, -)   class 2: (imag, -)   class 3: (-, -)
// so a complex key of 2w bits sorts in 2w/8 + 1 passes.  The reference sorts complex values
// with thrust and `less<complex>` (src/cupynumeric/sort/thrust_sort.h:129-145).
template <typename F>  // F = unsigned type of one component
struct ComplexOrder {
  F primary;
  F secondary;
  uint32_t cls;
};
template <typename F>
__host__ __device__ __forceinline__ ComplexOrder<F> complex_order(F real_bits, F imag_bits)
{
  constexpr F nan_key = static_cast<F>(~static_cast<F>(0));
  const F r           = ordered_bits<CODEC_FLOAT, F>(real_bits);
  const F i           = ordered_bits<CODEC_FLOAT, F>(imag_bits);
  const bool rn       = (r == nan_key);
  const bool in       = (i == nan_key);
  ComplexOrder<F> o;
  o.cls       = (rn ? 2u : 0u) + (in ? 1u : 0u);
  o.primary   = rn ? (in ? static_cast<F>(0) : i) : r;
  o.secondary = (rn || in) ? static_cast<F>(0) : i;
  return o;
}

template <>
struct KeyTraits<CODEC_COMPLEX, uint64_t> {  // complex64: real in the low, imag in the high 32 bits
  static constexpr int PASSES = 9;
  static constexpr int NWORDS = 2;
  static __host__ __device__ __forceinline__ void words(uint64_t raw, uint64_t (&w)[NWORDS])
  {
    const ComplexOrder<uint32_t> o =
      complex_order<uint32_t>(static_cast<uint32_t>(raw), static_cast<uint32_t>(raw >> 32));
    w[0] = (static_cast<uint64_t>(o.primary) << 32) | o.secondary;
    w[1] = o.cls;
  }
  static __host__ __device__ __forceinline__ uint32_t digit(uint64_t raw, int pass)
  {
    uint64_t w[NWORDS];
    words(raw, w);
    return pass < 8 ? static_cast<uint32_t>(w[0] >> (pass * 8)) & 0xFFu : static_cast<uint32_t>(w[1]);
  }
};

template <>
struct KeyTraits<CODEC_COMPLEX, U128> {  // complex128
  static constexpr int PASSES = 17;
  static constexpr int NWORDS = 3;
  static __host__ __device__ __forceinline__ void words(U128 raw, uint64_t (&w)[NWORDS])
  {
    const ComplexOrder<uint64_t> o = complex_order<uint64_t>(raw.lo, raw.hi);
    w[0]                           = o.secondary;
    w[1]                           = o.primary;
    w[2]                           = o.cls;
  }
  static __host__ __device__ __forceinline__ uint32_t digit(U128 raw, int pass)
  {
    uint64_t w[NWORDS];
    words(raw, w);
    const uint64_t v = pass < 8 ? w[0] : (pass < 16 ? w[1] : w[2]);
    return static_cast<uint32_t>(v >> ((pass & 7) * 8)) & 0xFFu;
  }
};

}  // namespace cpn
