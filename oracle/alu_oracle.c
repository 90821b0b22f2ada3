/*
 * alu_oracle.c -- CPU restatement of how the reference executes one Kernel.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing the product ships may call into this file; it exists so
 * that tests, the smoke check and the benchmark's CPU-baseline leg can compare the HIP path
 * against an independent evaluation of the same Kernel IR.
 *
 * What is restated, and from where (paths relative to the reference tree):
 *   - the dispatch loops of the interpreter backend              src/backend/cpu.ts:83-134
 *   - per-op semantics of AluExp.evaluate                        src/alu.ts:1059-1213
 *   - Reduction identity / fold                                  src/alu.ts:1584-1661
 *   - View index + validity arithmetic, multi-view chaining      src/shape.ts:277-300, 631-640, 690-700
 *   - the Wasm backend's lowering of each op (f32 arithmetic, logical shr, trunc_sat casts,
 *     float mod as a - trunc(a/b)*b, out-of-range loads read element 0)
 *                                                                src/backend/wasm/translation.ts:36-236
 *   - the Wasm backend's software transcendentals                src/backend/wasm/builtins.ts:25-494
 *   - threefry2x32 and the Abramowitz-Stegun erf                 src/alu.ts:1699-1793
 *
 * Two evaluation modes:
 *   JO_MODE_CPU  (0): the interpreter backend.  Floating-point values of every width are carried
 *                     as doubles and rounded once, on the store into the typed output
 *                     (src/backend/cpu.ts:121-132); transcendentals are libm's.
 *   JO_MODE_WASM (1): the Wasm backend.  Every f32 op rounds to f32, f64 ops stay in f64,
 *                     transcendentals are the reference's own polynomials evaluated in f32
 *                     (f64 arguments are demoted first, translation.ts:113-122).  The Wasm
 *                     backend has no float16 (translation.ts:558-586); for float16 nodes this
 *                     mode rounds after every op, which is how the reference's WebGPU backend
 *                     executes them, and calls transcendentals through the f32 polynomials.
 * Integer arithmetic wraps modulo 2^32 in both modes (the interpreter backend would go through
 * doubles, which only differs once a product exceeds 2^53).
 *
 * Pinning: tests/test_oracle_golden.py checks this file against every vector the reference's
 * own tests hold for the path (bit-op tables, cast/bitcast cases, NaN compares, saturating
 * casts, threefry known answers, erf values, view index cases, reductions with epilogues,
 * matmul shapes) and the software transcendentals against libm within the bounds the
 * reference asserts for them.  What only a live run of the reference could pin -- the exact
 * bits of f32 sums (order / fused multiply-add availability are engine dependent,
 * src/backend/wasm/codegen.ts:318-322) -- is compared with a tolerance, never bit for bit.
 */

#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

enum { JO_MODE_CPU = 0, JO_MODE_WASM = 1 };

enum { DT_F32 = 0, DT_I32 = 1, DT_U32 = 2, DT_BOOL = 3, DT_F16 = 4, DT_F64 = 5 };

enum {
  OP_ADD = 0, OP_SUB, OP_MUL, OP_IDIV, OP_MOD, OP_MIN, OP_MAX,
  OP_SIN, OP_COS, OP_ASIN, OP_ATAN, OP_EXP, OP_LOG, OP_ERF, OP_ERFC, OP_SQRT, OP_FLOOR, OP_CEIL,
  OP_RECIP, OP_CAST, OP_BITCAST,
  OP_BITCOMBINE, OP_BITINVERT, OP_BITSHIFT,
  OP_CMPLT, OP_CMPNE, OP_WHERE,
  OP_THREEFRY,
  OP_CONST, OP_SPECIAL, OP_VARIABLE, OP_GLOBALINDEX, OP_GLOBALVIEW
};

enum { VAR_GIDX = 0, VAR_RIDX = 1, VAR_ACC = 2 };

typedef struct {
  double d;  /* floating value (all float dtypes) */
  int64_t i; /* integer value: int32 sign-extended, uint32 zero-extended, bool 0/1 */
} jo_val;

typedef struct {
  int n;
  const int32_t *op, *dt, *soff, *src;
  const int64_t *ia; /* 2 per node */
  const double *fa;  /* 1 per node */
} jo_prog;

typedef struct {
  int mode;
  int nargs;
  const void *const *bufs;
  const int64_t *buf_bytes;
  const int64_t *views;
  int64_t oob; /* loads whose index fell outside the buffer */
  const char *err;
} jo_ctx;

static int is_float(int dt) { return dt == DT_F32 || dt == DT_F16 || dt == DT_F64; }
static int elem_bytes(int dt) { return dt == DT_F16 ? 2 : (dt == DT_F64 ? 8 : 4); }

#include "half.h" /* half_to_double, double_to_half */

static double round_dt(const jo_ctx *c, int dt, double x) {
  if (c->mode == JO_MODE_CPU) return x;
  if (dt == DT_F32) return (double)(float)x;
  if (dt == DT_F16) return half_to_double(double_to_half(x));
  return x;
}

static int64_t wrap_int(int dt, int64_t v) {
  if (dt == DT_I32) return (int64_t)(int32_t)(uint32_t)v;
  if (dt == DT_U32) return (int64_t)(uint32_t)v;
  return v != 0; /* bool */
}

/* ------------------------------------------- software transcendentals of the Wasm backend --- */

static float poly_f32(float x, const float *a, int n) {
  /* Horner, highest coefficient first; a zero coefficient skips its add (builtins.ts:6-17). */
  float r = a[n - 1];
  for (int i = n - 2; i >= 0; i--) {
    r = r * x;
    if (a[i] != 0.0f) r = r + a[i];
  }
  return r;
}

static int32_t trunc_sat_s(float x) {
  if (isnan(x)) return 0;
  if (x >= 2147483648.0f) return INT32_MAX;
  if (x <= -2147483648.0f) return INT32_MIN;
  return (int32_t)x;
}

static float wasm_exp(float x) { /* builtins.ts:25-90 */
  const float inv_ln2 = (float)(1.0 / 0.6931471805599453), ln2 = (float)0.6931471805599453;
  float kf = nearbyintf(x * inv_ln2);
  int32_t k = trunc_sat_s(kf);
  if (k > 127) return INFINITY;
  if (k < -126) return 0.0f;
  float r = x - kf * ln2;
  static const float a[7] = {1.0f, 1.0f, (float)(1.0 / 2), (float)(1.0 / 6), (float)(1.0 / 24),
                             (float)(1.0 / 120), (float)(1.0 / 720)};
  float p = poly_f32(r, a, 7);
  uint32_t bits = (uint32_t)(k + 127) << 23;
  float scale;
  memcpy(&scale, &bits, 4);
  return p * scale;
}

static float wasm_log(float x) { /* builtins.ts:99-193 */
  if (x < 0.0f) return NAN;
  uint32_t bits;
  memcpy(&bits, &x, 4);
  int32_t e = (int32_t)((bits >> 23) & 255) - 127;
  if (e == -127) return -INFINITY;
  if (e == 128) return x;
  uint32_t mb = (bits & 0x7fffff) | 0x3f800000;
  float m;
  memcpy(&m, &mb, 4);
  float t = (m - 1.0f) / (m + 1.0f);
  float t2 = t * t;
  static const float a[4] = {2.0f, (float)(2.0 / 3), (float)(2.0 / 5), (float)(2.0 / 7)};
  float lnm = poly_f32(t2, a, 4) * t;
  return (float)e * (float)0.6931471805599453 + lnm;
}

static void wasm_sincos(float x, int32_t *q, float *sz, float *cz) { /* builtins.ts:203-254 */
  const double PI = 3.141592653589793;
  float y = x - nearbyintf(x * (float)(1.0 / (2 * PI))) * (float)(2 * PI);
  float qf = nearbyintf(y * (float)(2 / PI));
  *q = trunc_sat_s(qf);
  float z = y - qf * (float)(PI / 2);
  float z2 = z * z;
  static const float s[4] = {1.0f, (float)(-1.0 / 6), (float)(1.0 / 120), (float)(-1.0 / 5040)};
  static const float c[5] = {1.0f, (float)(-1.0 / 2), (float)(1.0 / 24), (float)(-1.0 / 720), (float)(1.0 / 40320)};
  *sz = poly_f32(z2, s, 4) * z;
  *cz = poly_f32(z2, c, 5);
}

static float wasm_sin(float x) { /* builtins.ts:261-281 */
  int32_t q;
  float sz, cz;
  wasm_sincos(x, &q, &sz, &cz);
  float mag = (q & 1) ? cz : sz;
  return (q & 2) ? -mag : mag;
}

static float wasm_cos(float x) { /* builtins.ts:288-310 */
  int32_t q;
  float sz, cz;
  wasm_sincos(x, &q, &sz, &cz);
  float mag = (q & 1) ? sz : cz;
  return ((q + 1) & 2) ? -mag : mag;
}

static float wasm_atan(float x) { /* builtins.ts:313-392 */
  float ax = fabsf(x);
  float z = (ax >= 1.0f) ? 1.0f / ax : ax;
  float z2 = z * z;
  static const float P[3] = {(float)0.999998614341, (float)0.661705427875, (float)0.0415796528637};
  static const float Q[3] = {1.0f, (float)0.994987933645, (float)0.173698870181};
  float p = (poly_f32(z2, P, 3) / poly_f32(z2, Q, 3)) * z;
  float r = (ax >= 1.0f) ? (float)(3.141592653589793 / 2) - p : p;
  return copysignf(r, x);
}

static float wasm_asin(float x) { /* builtins.ts:399-415 */
  return wasm_atan(x / (1.0f + sqrtf(1.0f - x * x))) * 2.0f;
}

static float wasm_erfapprox(float x) { /* builtins.ts:422-455 */
  float t = 1.0f / (1.0f + (float)0.3275911 * x);
  static const float a[6] = {0.0f, (float)0.254829592, (float)-0.284496736, (float)1.421413741,
                             (float)-1.453152027, (float)1.061405429};
  return poly_f32(t, a, 6) * wasm_exp(-x * x);
}

static float wasm_erf(float x) { return copysignf(1.0f - wasm_erfapprox(fabsf(x)), x); }
static float wasm_erfc(float x) {
  float e = wasm_erfapprox(fabsf(x));
  return x < 0.0f ? 2.0f - e : e;
}

/* Abramowitz-Stegun 7.1.26 in double, as the interpreter backend evaluates it (alu.ts:1766-1793). */
static double js_erfapprox(double x) {
  double t = 1 / (1 + 0.3275911 * x);
  double P = ((((1.061405429 * t + -1.453152027) * t + 1.421413741) * t + -0.284496736) * t + 0.254829592) * t;
  return P * exp(-x * x);
}
static double js_erf(double x) { return x >= 0 ? 1 - js_erfapprox(x) : js_erfapprox(-x) - 1; }
static double js_erfc(double x) { return x >= 0 ? js_erfapprox(x) : 2 - js_erfapprox(-x); }

static void threefry2x32(uint32_t k0, uint32_t k1, uint32_t c0, uint32_t c1, uint32_t *o0, uint32_t *o1) {
  static const int rot[2][4] = {{13, 15, 26, 6}, {17, 29, 16, 24}};
  uint32_t ks[3] = {k0, k1, k0 ^ k1 ^ 0x1bd11bdaU};
  uint32_t x0 = c0 + ks[0], x1 = c1 + ks[1];
  for (int b = 0; b < 5; b++) {
    for (int j = 0; j < 4; j++) {
      int r = rot[b & 1][j];
      x0 += x1;
      x1 = ((x1 << r) | (x1 >> (32 - r))) ^ x0;
    }
    x0 += ks[(b + 1) % 3];
    x1 += ks[(b + 2) % 3] + (uint32_t)(b + 1);
  }
  *o0 = x0;
  *o1 = x1;
}

/* ------------------------------------------------------------------------ helpers ---------- */

static double js_min(double a, double b) {
  if (isnan(a) || isnan(b)) return NAN;
  if (a == 0 && b == 0) return signbit(a) ? a : b;
  return a < b ? a : b;
}
static double js_max(double a, double b) {
  if (isnan(a) || isnan(b)) return NAN;
  if (a == 0 && b == 0) return signbit(a) ? b : a;
  return a > b ? a : b;
}

static double unary_transcendental(const jo_ctx *c, int op, int dt, double x) {
  if (c->mode == JO_MODE_WASM) {
    float f = (float)x; /* f64 is demoted, f16/f32 widen exactly */
    float r;
    switch (op) {
      case OP_SIN: r = wasm_sin(f); break;
      case OP_COS: r = wasm_cos(f); break;
      case OP_ASIN: r = wasm_asin(f); break;
      case OP_ATAN: r = wasm_atan(f); break;
      case OP_EXP: r = wasm_exp(f); break;
      case OP_LOG: r = wasm_log(f); break;
      case OP_ERF: r = wasm_erf(f); break;
      default: r = wasm_erfc(f); break;
    }
    return round_dt(c, dt, (double)r);
  }
  switch (op) {
    case OP_SIN: return sin(x);
    case OP_COS: return cos(x);
    case OP_ASIN: return asin(x);
    case OP_ATAN: return atan(x);
    case OP_EXP: return exp(x);
    case OP_LOG: return log(x);
    case OP_ERF: return js_erf(x);
    default: return js_erfc(x);
  }
}

static double load_elem(jo_ctx *c, int gid, int dt, int64_t idx, int64_t *iout) {
  if (gid < 0 || gid >= c->nargs) {
    c->err = "gid out of bounds";
    return 0;
  }
  int64_t n = c->buf_bytes[gid] / elem_bytes(dt);
  if (idx < 0 || idx >= n) {
    c->oob++;
    idx = 0; /* translation.ts:221-228 reads element 0 instead of trapping */
    if (n == 0) {
      *iout = 0;
      return 0;
    }
  }
  const char *p = (const char *)c->bufs[gid];
  switch (dt) {
    case DT_F32: return (double)((const float *)p)[idx];
    case DT_F64: return ((const double *)p)[idx];
    case DT_F16: return half_to_double(((const uint16_t *)p)[idx]);
    case DT_I32: *iout = ((const int32_t *)p)[idx]; return 0;
    case DT_U32: *iout = ((const uint32_t *)p)[idx]; return 0;
    default: *iout = ((const int32_t *)p)[idx] != 0; return 0;
  }
}

/* Flat index + validity of a view chain (last view indexed by idx[], earlier ones by unravel). */
static int view_chain(const int64_t *vd, const int64_t *idx, int nidx, int64_t *flat_out) {
  int nviews = (int)vd[0];
  /* locate each view's record */
  const int64_t *rec[16];
  const int64_t *p = vd + 1;
  if (nviews > 16) return -1;
  for (int v = 0; v < nviews; v++) {
    rec[v] = p;
    int nd = (int)p[0], has_mask = (int)p[2];
    p += 3 + 2 * nd + (has_mask ? 2 * nd : 0);
  }
  int valid = 1;
  int64_t flat = 0;
  int64_t cur[16];
  for (int v = nviews - 1; v >= 0; v--) {
    const int64_t *r = rec[v];
    int nd = (int)r[0];
    int64_t off = r[1];
    int has_mask = (int)r[2];
    const int64_t *shape = r + 3, *strides = r + 3 + nd, *mask = r + 3 + 2 * nd;
    if (nd > 16) return -1;
    if (v == nviews - 1) {
      if (nidx != nd) return -1;
      for (int k = 0; k < nd; k++) cur[k] = idx[k];
    } else {
      int64_t acc = 1;
      for (int k = nd - 1; k >= 0; k--) { /* shape.ts:631-640: (flat / acc) % dim, C-style */
        int64_t d = shape[k];
        cur[k] = d ? (flat / acc) % d : 0;
        acc *= d;
      }
    }
    flat = off;
    for (int k = 0; k < nd; k++) {
      if (shape[k] != 1 && strides[k] != 0) flat += cur[k] * strides[k];
      if (has_mask && (cur[k] < mask[2 * k] || cur[k] >= mask[2 * k + 1])) valid = 0;
    }
  }
  *flat_out = flat;
  return valid;
}

/* ------------------------------------------------------------------------ evaluator -------- */

static void eval_prog(jo_ctx *c, const jo_prog *P, jo_val *v, int64_t gidx, int64_t ridx, const jo_val *acc) {
  for (int n = 0; n < P->n; n++) {
    const int op = P->op[n], dt = P->dt[n];
    const int32_t *s = P->src + P->soff[n];
    const int ns = P->soff[n + 1] - P->soff[n];
    jo_val r = {0, 0};
    switch (op) {
      case OP_ADD: case OP_SUB: case OP_MUL: case OP_IDIV: case OP_MOD: case OP_MIN: case OP_MAX: {
        const jo_val a = v[s[0]], b = v[s[1]];
        if (is_float(dt)) {
          double x = a.d, y = b.d, o;
          switch (op) {
            case OP_ADD: o = x + y; break;
            case OP_SUB: o = x - y; break;
            case OP_MUL: o = x * y; break;
            case OP_IDIV: o = trunc(round_dt(c, dt, x / y)); break;
            case OP_MOD:
              if (c->mode == JO_MODE_WASM) { /* a - trunc(a/b)*b, each step rounded */
                double q = trunc(round_dt(c, dt, x / y));
                o = x - round_dt(c, dt, q * y);
              } else {
                o = fmod(x, y);
              }
              break;
            case OP_MIN: o = js_min(x, y); break;
            default: o = js_max(x, y); break;
          }
          r.d = round_dt(c, dt, o);
        } else if (dt == DT_BOOL) {
          int x = a.i != 0, y = b.i != 0;
          switch (op) {
            case OP_ADD: case OP_MAX: r.i = x || y; break;
            case OP_MUL: case OP_MIN: r.i = x && y; break;
            case OP_SUB: r.i = (x - y) != 0; break;
            default: r.i = 0; break;
          }
        } else {
          int64_t x = a.i, y = b.i, o;
          switch (op) {
            case OP_ADD: o = x + y; break;
            case OP_SUB: o = x - y; break;
            case OP_MUL: o = (int64_t)((uint64_t)(uint32_t)x * (uint64_t)(uint32_t)y); break;
            case OP_IDIV: o = y == 0 ? 0 : x / y; break; /* Wasm traps on /0; the interpreter stores 0 */
            case OP_MOD: o = y == 0 ? 0 : x % y; break;
            case OP_MIN: o = x < y ? x : y; break;
            default: o = x > y ? x : y; break;
          }
          r.i = wrap_int(dt, o);
        }
        break;
      }
      case OP_SIN: case OP_COS: case OP_ASIN: case OP_ATAN: case OP_EXP: case OP_LOG: case OP_ERF: case OP_ERFC:
        r.d = unary_transcendental(c, op, dt, v[s[0]].d);
        break;
      case OP_SQRT: r.d = round_dt(c, dt, sqrt(v[s[0]].d)); break;
      case OP_FLOOR: r.d = floor(v[s[0]].d); break;
      case OP_CEIL: r.d = ceil(v[s[0]].d); break;
      case OP_RECIP: r.d = round_dt(c, dt, 1.0 / v[s[0]].d); break;
      case OP_CAST: {
        const int sdt = P->dt[s[0]];
        const jo_val a = v[s[0]];
        if (is_float(dt)) {
          r.d = round_dt(c, dt, is_float(sdt) ? a.d : (double)a.i);
        } else if (dt == DT_BOOL) {
          r.i = is_float(sdt) ? (a.d != 0) : (a.i != 0); /* NaN != 0 is true */
        } else if (is_float(sdt)) { /* saturating, NaN -> 0 (alu.ts:1128-1133, trunc_sat) */
          double x = a.d;
          if (isnan(x)) r.i = 0;
          else if (dt == DT_I32) r.i = x >= 2147483647.0 ? 2147483647LL : (x <= -2147483648.0 ? -2147483648LL : (int64_t)trunc(x));
          else r.i = x >= 4294967295.0 ? 4294967295LL : (x <= 0 ? 0 : (int64_t)trunc(x));
        } else {
          r.i = wrap_int(dt, a.i);
        }
        break;
      }
      case OP_BITCAST: {
        const int sdt = P->dt[s[0]];
        const jo_val a = v[s[0]];
        uint64_t bits = 0;
        if (sdt == DT_F32) { float f = (float)a.d; uint32_t u; memcpy(&u, &f, 4); bits = u; }
        else if (sdt == DT_F64) { memcpy(&bits, &a.d, 8); }
        else if (sdt == DT_F16) { bits = double_to_half(a.d); }
        else bits = (uint32_t)a.i;
        if (dt == DT_F32) { uint32_t u = (uint32_t)bits; float f; memcpy(&f, &u, 4); r.d = f; }
        else if (dt == DT_F64) { memcpy(&r.d, &bits, 8); }
        else if (dt == DT_F16) { r.d = half_to_double((uint16_t)bits); }
        else r.i = wrap_int(dt, (int64_t)bits);
        break;
      }
      case OP_BITCOMBINE: {
        uint32_t x = (uint32_t)v[s[0]].i, y = (uint32_t)v[s[1]].i, o;
        int m = (int)P->ia[2 * n];
        o = m == 0 ? (x & y) : (m == 1 ? (x | y) : (x ^ y));
        r.i = wrap_int(dt, (int64_t)o);
        break;
      }
      case OP_BITSHIFT: {
        uint32_t x = (uint32_t)v[s[0]].i, sh = (uint32_t)v[s[1]].i & 31u;
        uint32_t o = P->ia[2 * n] == 0 ? (x << sh) : (x >> sh); /* shr is logical for int32 too */
        r.i = wrap_int(dt, (int64_t)o);
        break;
      }
      case OP_CMPLT: {
        const int sdt = P->dt[s[0]];
        r.i = is_float(sdt) ? (v[s[0]].d < v[s[1]].d) : (v[s[0]].i < v[s[1]].i);
        break;
      }
      case OP_CMPNE: {
        const int sdt = P->dt[s[0]];
        r.i = is_float(sdt) ? (v[s[0]].d != v[s[1]].d) : (v[s[0]].i != v[s[1]].i);
        break;
      }
      case OP_WHERE: r = v[s[0]].i ? v[s[1]] : v[s[2]]; break;
      case OP_THREEFRY: {
        uint32_t o0, o1;
        threefry2x32((uint32_t)v[s[0]].i, (uint32_t)v[s[1]].i, (uint32_t)v[s[2]].i, (uint32_t)v[s[3]].i, &o0, &o1);
        int m = (int)P->ia[2 * n]; /* 2 = xor, 0 / 1 = word select */
        r.i = m == 2 ? (o0 ^ o1) : (m == 0 ? o0 : o1);
        break;
      }
      case OP_CONST:
        if (is_float(dt)) r.d = round_dt(c, dt, P->fa[n]);
        else r.i = P->ia[2 * n];
        break;
      case OP_SPECIAL: case OP_VARIABLE: {
        int which = (int)P->ia[2 * n];
        if (which == VAR_GIDX) r.i = gidx;
        else if (which == VAR_RIDX) r.i = ridx;
        else if (which == VAR_ACC && acc) r = *acc;
        else c->err = "unbound variable";
        break;
      }
      case OP_GLOBALINDEX:
        r.d = load_elem(c, (int)P->ia[2 * n], dt, v[s[0]].i, &r.i);
        break;
      case OP_GLOBALVIEW: {
        int64_t idx[16], flat = 0;
        if (ns > 16) { c->err = "too many view indices"; break; }
        for (int k = 0; k < ns; k++) idx[k] = v[s[k]].i;
        int valid = view_chain(c->views + P->ia[2 * n + 1], idx, ns, &flat);
        if (valid < 0) { c->err = "malformed view"; break; }
        if (valid) r.d = load_elem(c, (int)P->ia[2 * n], dt, flat, &r.i);
        break;
      }
      default: c->err = "unsupported op"; break;
    }
    v[n] = r;
  }
}

static jo_val reduce_identity(int op, int dt) { /* alu.ts:1584-1604 */
  jo_val r = {0, 0};
  if (dt == DT_BOOL) r.i = (op == OP_ADD || op == OP_MAX) ? 0 : 1;
  else if (dt == DT_I32) r.i = op == OP_ADD ? 0 : op == OP_MUL ? 1 : op == OP_MIN ? 2147483647LL : -2147483648LL;
  else if (dt == DT_U32) r.i = op == OP_ADD ? 0 : op == OP_MUL ? 1 : op == OP_MIN ? 4294967295LL : 0;
  else r.d = op == OP_ADD ? 0.0 : op == OP_MUL ? 1.0 : op == OP_MIN ? INFINITY : -INFINITY;
  return r;
}

static jo_val reduce_step(const jo_ctx *c, int op, int dt, jo_val a, jo_val b) { /* alu.ts:1607-1660 */
  jo_val r = {0, 0};
  if (dt == DT_BOOL) {
    r.i = (op == OP_ADD || op == OP_MAX) ? (a.i || b.i) : (a.i && b.i);
  } else if (is_float(dt)) {
    double o = op == OP_ADD ? a.d + b.d : op == OP_MUL ? a.d * b.d : op == OP_MIN ? js_min(a.d, b.d) : js_max(a.d, b.d);
    r.d = round_dt(c, dt, o);
  } else {
    int64_t o = op == OP_ADD ? a.i + b.i
              : op == OP_MUL ? (int64_t)((uint64_t)(uint32_t)a.i * (uint64_t)(uint32_t)b.i)
              : op == OP_MIN ? (a.i < b.i ? a.i : b.i) : (a.i > b.i ? a.i : b.i);
    r.i = wrap_int(dt, o);
  }
  return r;
}

static void store_elem(void *out, int dt, int64_t pos, jo_val x) {
  switch (dt) {
    case DT_F32: ((float *)out)[pos] = (float)x.d; break;
    case DT_F64: ((double *)out)[pos] = x.d; break;
    case DT_F16: ((uint16_t *)out)[pos] = double_to_half(x.d); break;
    case DT_U32: ((uint32_t *)out)[pos] = (uint32_t)x.i; break;
    default: ((int32_t *)out)[pos] = (int32_t)x.i; break;
  }
}

/*
 * Evaluate a kernel.  rsize < 0 means "no reduction".  When gidx_list is non-NULL only those
 * output positions are computed and they are written densely (out[k] for gidx_list[k]).
 * Returns 0 on success; *oob_out receives the number of out-of-range loads.
 */
int jo_run_kernel(int mode, int64_t size, int64_t rsize, int red_op, int red_dt,
                  int n_exp, const int32_t *e_op, const int32_t *e_dt, const int32_t *e_soff, const int32_t *e_src,
                  const int64_t *e_ia, const double *e_fa,
                  int n_epi, const int32_t *p_op, const int32_t *p_dt, const int32_t *p_soff, const int32_t *p_src,
                  const int64_t *p_ia, const double *p_fa,
                  const int64_t *views, int nargs, const void *const *bufs, const int64_t *buf_bytes,
                  void *out, int out_dt, const int64_t *gidx_list, int64_t n_list, int64_t *oob_out,
                  char *err, int errlen) {
  jo_prog E = {n_exp, e_op, e_dt, e_soff, e_src, e_ia, e_fa};
  jo_prog P = {n_epi, p_op, p_dt, p_soff, p_src, p_ia, p_fa};
  jo_ctx c = {mode, nargs, bufs, buf_bytes, views, 0, NULL};
  jo_val *ve = (jo_val *)calloc((size_t)(n_exp > 0 ? n_exp : 1), sizeof(jo_val));
  jo_val *vp = (jo_val *)calloc((size_t)(n_epi > 0 ? n_epi : 1), sizeof(jo_val));
  if (!ve || !vp) {
    snprintf(err, (size_t)errlen, "out of memory");
    free(ve);
    free(vp);
    return 1;
  }
  const int64_t count = gidx_list ? n_list : size;
  for (int64_t k = 0; k < count && !c.err; k++) {
    const int64_t g = gidx_list ? gidx_list[k] : k;
    jo_val res;
    if (rsize < 0) {
      eval_prog(&c, &E, ve, g, 0, NULL);
      res = ve[n_exp - 1];
    } else {
      jo_val acc = reduce_identity(red_op, red_dt);
      for (int64_t j = 0; j < rsize && !c.err; j++) {
        eval_prog(&c, &E, ve, g, j, NULL);
        acc = reduce_step(&c, red_op, red_dt, acc, ve[n_exp - 1]);
      }
      eval_prog(&c, &P, vp, g, 0, &acc);
      res = vp[n_epi - 1];
    }
    store_elem(out, out_dt, k, res);
  }
  free(ve);
  free(vp);
  if (oob_out) *oob_out = c.oob;
  if (c.err) {
    snprintf(err, (size_t)errlen, "%s", c.err);
    return 1;
  }
  return 0;
}

/* Scalar entry points so the builtins can be pinned one function at a time. */
float jo_wasm_exp(float x) { return wasm_exp(x); }
float jo_wasm_log(float x) { return wasm_log(x); }
float jo_wasm_sin(float x) { return wasm_sin(x); }
float jo_wasm_cos(float x) { return wasm_cos(x); }
float jo_wasm_atan(float x) { return wasm_atan(x); }
float jo_wasm_asin(float x) { return wasm_asin(x); }
float jo_wasm_erf(float x) { return wasm_erf(x); }
float jo_wasm_erfc(float x) { return wasm_erfc(x); }
double jo_js_erf(double x) { return js_erf(x); }
double jo_js_erfc(double x) { return js_erfc(x); }
void jo_threefry2x32(uint32_t k0, uint32_t k1, uint32_t c0, uint32_t c1, uint32_t *out2) {
  threefry2x32(k0, k1, c0, c1, out2, out2 + 1);
}
uint16_t jo_double_to_half(double x) { return double_to_half(x); }
double jo_half_to_double(uint16_t h) { return half_to_double(h); }
