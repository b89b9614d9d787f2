/*
 * TEST INFRASTRUCTURE ONLY. Scalar types and conversions for the CPU oracle.
 *
 * The oracle restates the arithmetic of the reference's CPU path
 * (csrc/cpu/reducer.h:43-84) in plain C. Half and BFloat16 are carried as
 * 16-bit patterns; every arithmetic step on them goes through float and is
 * rounded back with round-to-nearest-even, which is what c10::Half and
 * c10::BFloat16 operators do.
 */
#ifndef TS_ORACLE_TYPES_H
#define TS_ORACLE_TYPES_H

#include <stdint.h>
#include <string.h>

/* dtype codes (shared with the HIP C-ABI) */
enum { TSO_F32 = 0, TSO_F64 = 1, TSO_F16 = 2, TSO_BF16 = 3, TSO_I32 = 4,
       TSO_I64 = 5, TSO_I16 = 6, TSO_I8 = 7, TSO_U8 = 8 };

/* reduce codes: same order as the reference enum (csrc/cpu/reducer.h:6) */
enum { TSO_SUM = 0, TSO_MEAN = 1, TSO_MUL = 2, TSO_DIV = 3, TSO_MIN = 4,
       TSO_MAX = 5 };

typedef struct { uint16_t x; } tso_half;
typedef struct { uint16_t x; } tso_bf16;

static inline float tso_bits_to_float(uint32_t u) {
  float f;
  memcpy(&f, &u, 4);
  return f;
}
static inline uint32_t tso_float_to_bits(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  return u;
}

/* bf16 -> float: the pattern is the high half of the float */
static inline float tso_bf16_to_float(tso_bf16 h) {
  return tso_bits_to_float((uint32_t)h.x << 16);
}
/* float -> bf16, round to nearest even; NaN maps to 0x7FC0 */
static inline tso_bf16 tso_float_to_bf16(float f) {
  tso_bf16 r;
  uint32_t u = tso_float_to_bits(f);
  if ((u & 0x7FFFFFFFu) > 0x7F800000u) {
    r.x = 0x7FC0;
    return r;
  }
  uint32_t bias = 0x7FFFu + ((u >> 16) & 1u);
  r.x = (uint16_t)((u + bias) >> 16);
  return r;
}

/* IEEE binary16 -> float */
static inline float tso_half_to_float(tso_half h) {
  uint32_t sign = ((uint32_t)h.x & 0x8000u) << 16;
  uint32_t exp = (h.x >> 10) & 0x1Fu;
  uint32_t man = h.x & 0x3FFu;
  uint32_t u;
  if (exp == 0) {
    if (man == 0) {
      u = sign;
    } else { /* subnormal: normalise */
      int e = -1;
      do {
        man <<= 1;
        e++;
      } while (!(man & 0x400u));
      man &= 0x3FFu;
      u = sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13);
    }
  } else if (exp == 31) {
    u = sign | 0x7F800000u | (man << 13);
  } else {
    u = sign | ((exp + 127 - 15) << 23) | (man << 13);
  }
  return tso_bits_to_float(u);
}

/* float -> IEEE binary16, round to nearest even */
static inline tso_half tso_float_to_half(float f) {
  tso_half r;
  uint32_t u = tso_float_to_bits(f);
  uint32_t sign = (u >> 16) & 0x8000u;
  uint32_t a = u & 0x7FFFFFFFu;
  if (a > 0x7F800000u) { /* NaN */
    r.x = (uint16_t)(sign | 0x7E00u);
    return r;
  }
  if (a >= 0x47800000u) { /* >= 65536 (incl. inf): overflow to inf */
    r.x = (uint16_t)(sign | 0x7C00u);
    return r;
  }
  if (a < 0x33000001u) { /* <= 2^-25: rounds to zero */
    r.x = (uint16_t)sign;
    return r;
  }
  int32_t e = (int32_t)(a >> 23) - 127;
  uint32_t m = (a & 0x7FFFFFu) | 0x800000u; /* 24-bit significand */
  uint32_t shift, half;
  uint32_t out;
  if (e < -14) { /* subnormal half: value = m * 2^(e-23), unit 2^-24 */
    shift = (uint32_t)(-e - 1); /* 14..24: (e-23)+24 = e+1 -> shift = -(e+1) */
    out = m >> shift;
    half = 1u << (shift - 1);
    uint32_t rem = m & ((1u << shift) - 1u);
    if (rem > half || (rem == half && (out & 1u)))
      out++;
    r.x = (uint16_t)(sign | out);
    return r;
  }
  /* normal: keep 10 fraction bits */
  out = ((uint32_t)(e + 15) << 10) | ((m >> 13) & 0x3FFu);
  uint32_t rem = m & 0x1FFFu;
  if (rem > 0x1000u || (rem == 0x1000u && (out & 1u)))
    out++; /* carry may bump the exponent; 0x7C00 (inf) is then correct */
  r.x = (uint16_t)(sign | out);
  return r;
}

#endif
