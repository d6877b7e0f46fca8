// Fixed-point requantisation arithmetic shared by host (Prepare-time derivation) and device (epilogues) code.
// Semantics follow nnacl's gemmlowp-style helpers (reference: mindspore/ccsrc/plugin/device/cpu/kernel/nnacl/int8/
// fixed_point.c:26-68 and quantize.c:39-161); the formulations here are branch-light equivalents suited to VALU code.
#pragma once

#include <stdint.h>

#if defined(__HIPCC__)
#define MI_HD __host__ __device__ __forceinline__
#else
#define MI_HD inline
#endif

namespace mi {

// SaturatingRoundingDoublingHighMul: floor((a*b + 2^30) / 2^31); ties toward +inf; saturates only for
// a == b == INT32_MIN.  The 64-bit sum cannot overflow (|a*b| <= 2^62).
MI_HD int32_t srdhm(int32_t a, int32_t b) {
  const int64_t p = (int64_t)a * (int64_t)b + ((int64_t)1 << 30);
  const int32_t r = (int32_t)(p >> 31);  // arithmetic shift == floor division
  return (a == INT32_MIN && b == INT32_MIN) ? INT32_MAX : r;
}

// Same without the saturation test: valid whenever b != INT32_MIN.
MI_HD int32_t srdhm_nosat(int32_t a, int32_t b) {
  const int64_t p = (int64_t)a * (int64_t)b + ((int64_t)1 << 30);
  return (int32_t)(p >> 31);
}

// RoundingDivideByPOT for 0 <= e <= 31: round to nearest, ties away from zero.
MI_HD int32_t rdiv_pot(int32_t x, int32_t e) {
  const int32_t mask = (int32_t)(((uint32_t)1 << e) - 1u);  // e == 31 -> 0x7fffffff
  const int32_t rem = x & mask;
  const int32_t thr = (mask >> 1) + (x < 0 ? 1 : 0);
  return (x >> e) + (rem > thr ? 1 : 0);
}

// Same for 1 <= e <= 30 when x + 2^(e-1) cannot overflow int32: (x + half - (x < 0)) >> e.
MI_HD int32_t rdiv_pot_fast(int32_t x, int32_t e, int32_t half) { return (x + half + (x >> 31)) >> e; }

// MultiplyByQuantizedMultiplier: the pre-shift wraps in int32; rs <= 0.
MI_HD int32_t mul_by_quant_mult(int32_t v, int32_t mult, int32_t ls, int32_t rs) {
  const int32_t shifted = (int32_t)((uint32_t)v << ls);
  const int32_t e = -rs > 31 ? 31 : -rs;
  return rdiv_pot(srdhm(shifted, mult), e);
}

}  // namespace mi
