// =================================================================================================
// Host-side fp16 <-> fp32 conversion with the semantics of CLBlast's `include/clblast_half.h`
// (reference: FloatToHalf :34-97, HalfToFloat :101-347), written as branch arithmetic rather than
// lookup tables. Pure C99, header-only.
//
//   FloatToHalf: truncation (round toward zero). Magnitudes >= 2^16 (including values that IEEE
//                round-to-nearest would keep finite) become infinity; magnitudes < 2^-24 become
//                signed zero; subnormal halves are produced by shifting the mantissa *without* the
//                implicit leading one being rounded (plain truncation); NaN keeps its top 10 mantissa
//                bits (a NaN whose top 10 mantissa bits are zero turns into infinity).
//   HalfToFloat: exact (every binary16 value is representable in binary32).
// =================================================================================================
#ifndef CLBLAST_HIP_HALF_H_
#define CLBLAST_HIP_HALF_H_

#include <string.h>

// The host type for half precision is the IEEE binary16 bit pattern (reference: clblast_half.h:21).
typedef unsigned short half;

static inline half FloatToHalf(const float value) {
  unsigned int bits;
  memcpy(&bits, &value, sizeof(bits));
  const unsigned int sign = (bits >> 16) & 0x8000u;
  const int exponent = (int)((bits >> 23) & 0xFFu) - 127;  // unbiased
  const unsigned int mantissa = bits & 0x7FFFFFu;
  if (exponent < -24) {  // too small even for a subnormal half
    return (half)sign;
  }
  if (exponent < -14) {  // subnormal half: leading one at bit (24 + exponent), mantissa bits below it
    const unsigned int leading = 0x0400u >> (unsigned)(-exponent - 14);
    return (half)(sign + leading + (mantissa >> (unsigned)(-exponent - 1)));
  }
  if (exponent <= 15) {  // normal half
    return (half)(sign + ((unsigned)(exponent + 15) << 10) + (mantissa >> 13));
  }
  if (exponent < 128) {  // finite float beyond the half range: infinity
    return (half)(sign + 0x7C00u);
  }
  return (half)(sign + 0x7C00u + (mantissa >> 13));  // infinity and NaN
}

static inline float HalfToFloat(const half value) {
  const unsigned int sign = ((unsigned int)value & 0x8000u) << 16;
  unsigned int exponent = ((unsigned int)value >> 10) & 0x1Fu;
  unsigned int mantissa = (unsigned int)value & 0x3FFu;
  unsigned int bits;
  if (exponent == 0) {
    if (mantissa == 0) {
      bits = sign;  // signed zero
    } else {        // subnormal half: normalise
      int e = -1;
      do {
        mantissa <<= 1;
        ++e;
      } while ((mantissa & 0x400u) == 0);
      bits = sign | ((unsigned)(112 - e) << 23) | ((mantissa & 0x3FFu) << 13);
    }
  } else if (exponent == 31) {
    bits = sign | 0x7F800000u | (mantissa << 13);  // infinity / NaN
  } else {
    bits = sign | ((exponent + 112u) << 23) | (mantissa << 13);
  }
  float result;
  memcpy(&result, &bits, sizeof(result));
  return result;
}

#endif  // CLBLAST_HIP_HALF_H_
