/* TEST INFRASTRUCTURE ONLY. Exposes the reference's own fp16 conversion routines (include/clblast_half.h
 * in the CLBlast tree, included from where it lies; nothing is copied) so that the tests can compare
 * the oracle's and the library's conversions with them bit for bit. Built into oracle/_ref/ by
 * oracle/Makefile when the reference tree is present. */
#include "clblast_half.h"

__attribute__((visibility("default"))) unsigned short ref_float_to_half(float value) { return FloatToHalf(value); }
__attribute__((visibility("default"))) float ref_half_to_float(unsigned short value) { return HalfToFloat(value); }
