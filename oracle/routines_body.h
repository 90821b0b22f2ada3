/* Bodies of the dense routines of routines_oracle.c for one element type.  TEST INFRASTRUCTURE ONLY.
 *
 * Included once per element type with
 *   RO_T        storage type of an element (float, double, uint16_t holding a float16)
 *   RO_LD(x)    the element as a double (what reading a typed array gives JavaScript)
 *   RO_ST(v)    a double rounded to the element type (what a typed-array store does)
 *   RO_NAME(f)  the function's name for this type
 * Every scalar in between is a double, as in the reference. */

void RO_NAME(ro_triangular_solve)(const RO_T* a, const RO_T* b, RO_T* x, int64_t mats, int64_t batch, int64_t n, int unit_diagonal) {
  for (int64_t counter = 0; counter < mats; counter++) {
    const RO_T* a1 = a + counter * n * n;
    for (int64_t t = 0; t < batch; t++) {
      const RO_T* b1 = b + (counter * batch + t) * n;
      RO_T* x1 = x + (counter * batch + t) * n;
      for (int64_t i = n - 1; i >= 0; i--) {
        double sum = RO_LD(b1[i]);
        for (int64_t j = i + 1; j < n; j++) sum -= RO_LD(a1[i * n + j]) * RO_LD(x1[j]);
        x1[i] = unit_diagonal ? RO_ST(sum) : RO_ST(sum / RO_LD(a1[i * n + i]));
      }
    }
  }
}

void RO_NAME(ro_cholesky)(const RO_T* x, RO_T* y, int64_t mats, int64_t n) {
  memset(y, 0, sizeof(RO_T) * (size_t)(mats * n * n));
  for (int64_t m = 0; m < mats; m++) {
    const RO_T* ar = x + m * n * n;
    RO_T* out = y + m * n * n;
    for (int64_t i = 0; i < n; i++) {
      for (int64_t j = 0; j <= i; j++) {
        double sum = RO_LD(ar[i * n + j]);
        for (int64_t k = 0; k < j; k++) sum -= RO_LD(out[i * n + k]) * RO_LD(out[j * n + k]);
        out[i * n + j] = i == j ? RO_ST(sqrt(sum)) : RO_ST(sum / RO_LD(out[j * n + j]));
      }
    }
  }
}

void RO_NAME(ro_lu)(const RO_T* a, RO_T* lu, int32_t* pivots, int32_t* perm, int64_t mats, int64_t m, int64_t n) {
  const int64_t r = m < n ? m : n;
  for (int64_t b = 0; b < mats; b++) {
    const RO_T* ar = a + b * m * n;
    RO_T* out = lu + b * m * n;
    int32_t* piv = pivots + b * r;
    int32_t* p = perm + b * m;
    memcpy(out, ar, sizeof(RO_T) * (size_t)(m * n));
    for (int64_t i = 0; i < m; i++) p[i] = (int32_t)i;
    for (int64_t j = 0; j < r; j++) {
      double max_val = fabs(RO_LD(out[j * n + j]));
      int64_t max_row = j;
      for (int64_t i = j + 1; i < m; i++) {
        const double val = fabs(RO_LD(out[i * n + j]));
        if (val > max_val) {
          max_val = val;
          max_row = i;
        }
      }
      piv[j] = (int32_t)max_row;
      if (max_row != j) {
        for (int64_t col = 0; col < n; col++) {
          const RO_T tmp = out[j * n + col];
          out[j * n + col] = out[max_row * n + col];
          out[max_row * n + col] = tmp;
        }
        const int32_t tp = p[j];
        p[j] = p[max_row];
        p[max_row] = tp;
      }
      const double diag = RO_LD(out[j * n + j]);
      if (diag != 0) {
        for (int64_t i = j + 1; i < m; i++) {
          const double factor = RO_LD(out[i * n + j]) / diag;
          out[i * n + j] = RO_ST(factor);
          for (int64_t col = j + 1; col < n; col++) out[i * n + col] = RO_ST(RO_LD(out[i * n + col]) - factor * RO_LD(out[j * n + col]));
        }
      }
    }
  }
}

void RO_NAME(ro_jacobi_eigh)(const RO_T* input, RO_T* diagonalized, RO_T* vectors, int64_t mats, int64_t n, int64_t max_sweeps, double tolerance) {
  for (int64_t mat = 0; mat < mats; mat++) {
    const RO_T* x = input + mat * n * n;
    RO_T* a = diagonalized + mat * n * n;
    RO_T* v = vectors + mat * n * n;
    memset(a, 0, sizeof(RO_T) * (size_t)(n * n));
    for (int64_t i = 0; i < n; i++)
      for (int64_t j = 0; j <= i; j++) a[i * n + j] = x[i * n + j];
    memset(v, 0, sizeof(RO_T) * (size_t)(n * n));
    for (int64_t i = 0; i < n; i++) v[i * n + i] = RO_ST(1.0);
    double max_abs = 1;
    for (int64_t i = 0; i < n; i++)
      for (int64_t j = 0; j <= i; j++) max_abs = js_max(max_abs, fabs(RO_LD(a[i * n + j])));
    const double threshold = tolerance * max_abs;
#define SYM(i, j) ((i) >= (j) ? (i) * n + (j) : (j) * n + (i))
#define MAX_OFF(dst)                                                                  \
  do {                                                                                \
    dst = 0;                                                                          \
    for (int64_t i_ = 0; i_ < n; i_++)                                                \
      for (int64_t j_ = 0; j_ < i_; j_++) dst = js_max(dst, fabs(RO_LD(a[i_ * n + j_]))); \
  } while (0)
    double max_off;
    MAX_OFF(max_off);
    for (int64_t sweep = 0; sweep < max_sweeps && max_off > threshold; sweep++) {
      for (int64_t p = 0; p < n - 1; p++) {
        for (int64_t q = p + 1; q < n; q++) {
          const int64_t pp = p * n + p, qq = q * n + q, pq = SYM(p, q);
          const double app = RO_LD(a[pp]), aqq = RO_LD(a[qq]), apq = RO_LD(a[pq]);
          if (apq == 0) continue;
          const double tau = (aqq - app) / (2 * apq);
          const double tau_sign = tau >= 0 ? 1 : -1;
          const double t = tau_sign / (fabs(tau) + sqrt(tau * tau + 1));
          const double c = 1 / sqrt(t * t + 1);
          const double s = t * c;
          for (int64_t k = 0; k < n; k++) {
            if (k == p || k == q) continue;
            const int64_t kp = SYM(k, p), kq = SYM(k, q);
            const double akp = RO_LD(a[kp]), akq = RO_LD(a[kq]);
            const double next_kp = c * akp - s * akq;
            const double next_kq = s * akp + c * akq;
            a[kp] = RO_ST(next_kp);
            a[kq] = RO_ST(next_kq);
          }
          a[pp] = RO_ST(c * c * app - 2 * s * c * apq + s * s * aqq);
          a[qq] = RO_ST(s * s * app + 2 * s * c * apq + c * c * aqq);
          a[pq] = RO_ST(0.0);
          for (int64_t k = 0; k < n; k++) {
            const int64_t kp = k * n + p, kq = k * n + q;
            const double vkp = RO_LD(v[kp]), vkq = RO_LD(v[kq]);
            v[kp] = RO_ST(c * vkp - s * vkq);
            v[kq] = RO_ST(s * vkp + c * vkq);
          }
        }
      }
      MAX_OFF(max_off);
    }
#undef SYM
#undef MAX_OFF
  }
}

int RO_NAME(ro_fft)(const RO_T* real, const RO_T* imag, RO_T* out_real, RO_T* out_imag, int64_t rows, int64_t n, const int32_t* factors,
                    int32_t nfactors, int inverse) {
  const double angle_scale = (inverse ? 2 : -2) * 3.141592653589793;
  uint32_t* permutation = (uint32_t*)malloc(sizeof(uint32_t) * (size_t)(n > 0 ? n : 1));
  int32_t max_factor = 1;
  for (int32_t f = 0; f < nfactors; f++)
    if (factors[f] > max_factor) max_factor = factors[f];
  double* scratch_real = (double*)malloc(sizeof(double) * (size_t)max_factor);
  double* scratch_imag = (double*)malloc(sizeof(double) * (size_t)max_factor);
  if (!permutation || !scratch_real || !scratch_imag) return 1;
  for (int64_t index = 0; index < n; index++) {
    int64_t remaining = index, stride = 1, reversed = 0;
    for (int32_t f = 0; f < nfactors; f++) {
      const int64_t digit = remaining % factors[f];
      remaining = remaining / factors[f];
      stride *= factors[f];
      reversed += digit * (n / stride);
    }
    permutation[index] = (uint32_t)reversed;
  }
  for (int64_t row = 0; row < rows; row++) {
    const int64_t offset = row * n;
    for (int64_t index = 0; index < n; index++) {
      out_real[offset + index] = real[offset + permutation[index]];
      out_imag[offset + index] = imag[offset + permutation[index]];
    }
    int64_t prev = 1;
    for (int32_t stage = 0; stage < nfactors; stage++) {
      const int64_t radix = factors[stage];
      const int64_t span = prev * radix;
      const double stage_scale = inverse && stage == nfactors - 1 ? 1.0 / (double)n : 1;
      for (int64_t group = 0; group < n; group += span) {
        for (int64_t j = 0; j < prev; j++) {
          for (int64_t q = 0; q < radix; q++) {
            const int64_t idx = offset + group + j + q * prev;
            const double angle = (angle_scale * (double)q * (double)j) / (double)span;
            const double c = cos(angle), s = sin(angle);
            const double xr = RO_LD(out_real[idx]), xi = RO_LD(out_imag[idx]);
            scratch_real[q] = xr * c - xi * s;
            scratch_imag[q] = xr * s + xi * c;
          }
          for (int64_t p = 0; p < radix; p++) {
            double sum_real = 0, sum_imag = 0;
            for (int64_t q = 0; q < radix; q++) {
              const double angle = (angle_scale * (double)q * (double)p) / (double)radix;
              const double c = cos(angle), s = sin(angle);
              const double xr = scratch_real[q], xi = scratch_imag[q];
              sum_real += xr * c - xi * s;
              sum_imag += xr * s + xi * c;
            }
            const int64_t idx = offset + group + j + p * prev;
            out_real[idx] = RO_ST(sum_real * stage_scale);
            out_imag[idx] = RO_ST(sum_imag * stage_scale);
          }
        }
      }
      prev = span;
    }
  }
  free(permutation);
  free(scratch_real);
  free(scratch_imag);
  return 0;
}
