/* float16 <-> double for the CPU checkers.  TEST INFRASTRUCTURE ONLY (see alu_oracle.c, routines_oracle.c).
 * A Float16Array store rounds the double to nearest-even in one step; so does double_to_half. */
#ifndef ORACLE_HALF_H
#define ORACLE_HALF_H
#include <math.h>
#include <stdint.h>
#include <string.h>

static inline double half_to_double(uint16_t h) {
  int sign = h >> 15, e = (h >> 10) & 31, m = h & 1023;
  double v;
  if (e == 0) v = ldexp((double)m, -24);
  else if (e == 31) v = m ? NAN : INFINITY;
  else v = ldexp((double)(m | 1024), e - 25);
  return sign ? -v : v;
}

/* Round-to-nearest-even straight from double, so no double rounding through float. */
static inline uint16_t double_to_half(double x) {
  uint64_t b;
  memcpy(&b, &x, 8);
  uint16_t sign = (uint16_t)((b >> 48) & 0x8000);
  int e = (int)((b >> 52) & 0x7ff);
  uint64_t m = b & 0xfffffffffffffULL;
  if (e == 0x7ff) return (uint16_t)(sign | 0x7c00 | (m ? 0x200 : 0));
  if (e == 0) return sign; /* double subnormals are far below half's range */
  int E = e - 1023;
  if (E > 15) return (uint16_t)(sign | 0x7c00);
  uint64_t sig = m | (1ULL << 52);
  int shift = E >= -14 ? 42 : 42 + (-14 - E);
  if (shift > 54) return sign;
  uint64_t q = sig >> shift, rem = sig & ((1ULL << shift) - 1), half = 1ULL << (shift - 1);
  if (rem > half || (rem == half && (q & 1))) q++;
  uint32_t h = E >= -14 ? (uint32_t)(((uint32_t)(E + 14) << 10) + q) : (uint32_t)q;
  if (h >= 0x7c00) h = 0x7c00;
  return (uint16_t)(sign | h);
}

#endif
