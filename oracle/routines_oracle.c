/* CPU restatement of the reference's dense routines for float32 operands.  TEST INFRASTRUCTURE ONLY: the
 * product never links or calls this file; it is the checker the GPU kernels are compared with.
 *
 * Every function follows the loop structure of the reference's CPU implementation and keeps its arithmetic:
 * scalars are doubles (JavaScript numbers), typed-array stores round to float32.  Built with
 * -ffp-contract=off so that no multiply-add is fused.
 *
 *   ro_triangular_solve  src/routine.ts:298-336
 *   ro_cholesky          src/routine.ts:338-362
 *   ro_lu                src/routine.ts:364-420
 *   ro_jacobi_eigh       src/routine.ts:422-543
 *   ro_fft               src/routine.ts:545-640
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

void ro_triangular_solve(const float* a, const float* b, float* x, int64_t mats, int64_t batch, int64_t n, int unit_diagonal) {
  for (int64_t counter = 0; counter < mats; counter++) {
    const float* a1 = a + counter * n * n;
    for (int64_t t = 0; t < batch; t++) {
      const float* b1 = b + (counter * batch + t) * n;
      float* x1 = x + (counter * batch + t) * n;
      for (int64_t i = n - 1; i >= 0; i--) {
        double sum = b1[i];
        for (int64_t j = i + 1; j < n; j++) sum -= (double)a1[i * n + j] * (double)x1[j];
        x1[i] = unit_diagonal ? (float)sum : (float)(sum / (double)a1[i * n + i]);
      }
    }
  }
}

void ro_cholesky(const float* x, float* y, int64_t mats, int64_t n) {
  memset(y, 0, sizeof(float) * (size_t)(mats * n * n));
  for (int64_t m = 0; m < mats; m++) {
    const float* ar = x + m * n * n;
    float* out = y + m * n * n;
    for (int64_t i = 0; i < n; i++) {
      for (int64_t j = 0; j <= i; j++) {
        double sum = ar[i * n + j];
        for (int64_t k = 0; k < j; k++) sum -= (double)out[i * n + k] * (double)out[j * n + k];
        out[i * n + j] = i == j ? (float)sqrt(sum) : (float)(sum / (double)out[j * n + j]);
      }
    }
  }
}

void ro_lu(const float* a, float* lu, int32_t* pivots, int32_t* perm, int64_t mats, int64_t m, int64_t n) {
  const int64_t r = m < n ? m : n;
  for (int64_t b = 0; b < mats; b++) {
    const float* ar = a + b * m * n;
    float* out = lu + b * m * n;
    int32_t* piv = pivots + b * r;
    int32_t* p = perm + b * m;
    memcpy(out, ar, sizeof(float) * (size_t)(m * n));
    for (int64_t i = 0; i < m; i++) p[i] = (int32_t)i;
    for (int64_t j = 0; j < r; j++) {
      double max_val = fabs((double)out[j * n + j]);
      int64_t max_row = j;
      for (int64_t i = j + 1; i < m; i++) {
        const double val = fabs((double)out[i * n + j]);
        if (val > max_val) {
          max_val = val;
          max_row = i;
        }
      }
      piv[j] = (int32_t)max_row;
      if (max_row != j) {
        for (int64_t col = 0; col < n; col++) {
          const float tmp = out[j * n + col];
          out[j * n + col] = out[max_row * n + col];
          out[max_row * n + col] = tmp;
        }
        const int32_t tp = p[j];
        p[j] = p[max_row];
        p[max_row] = tp;
      }
      const double diag = out[j * n + j];
      if (diag != 0) {
        for (int64_t i = j + 1; i < m; i++) {
          const double factor = (double)out[i * n + j] / diag;
          out[i * n + j] = (float)factor;
          for (int64_t col = j + 1; col < n; col++) out[i * n + col] = (float)((double)out[i * n + col] - factor * (double)out[j * n + col]);
        }
      }
    }
  }
}

static double js_max(double a, double b) { return (a != a || b != b) ? NAN : (a > b ? a : b); }

void ro_jacobi_eigh(const float* input, float* diagonalized, float* vectors, int64_t mats, int64_t n, int64_t max_sweeps, double tolerance) {
  for (int64_t mat = 0; mat < mats; mat++) {
    const float* x = input + mat * n * n;
    float* a = diagonalized + mat * n * n;
    float* v = vectors + mat * n * n;
    memset(a, 0, sizeof(float) * (size_t)(n * n));
    for (int64_t i = 0; i < n; i++)
      for (int64_t j = 0; j <= i; j++) a[i * n + j] = x[i * n + j];
    memset(v, 0, sizeof(float) * (size_t)(n * n));
    for (int64_t i = 0; i < n; i++) v[i * n + i] = 1.0f;
    double max_abs = 1;
    for (int64_t i = 0; i < n; i++)
      for (int64_t j = 0; j <= i; j++) max_abs = js_max(max_abs, fabs((double)a[i * n + j]));
    const double threshold = tolerance * max_abs;
#define SYM(i, j) ((i) >= (j) ? (i) * n + (j) : (j) * n + (i))
#define MAX_OFF(dst)                                                                   \
  do {                                                                                 \
    dst = 0;                                                                           \
    for (int64_t i_ = 0; i_ < n; i_++)                                                 \
      for (int64_t j_ = 0; j_ < i_; j_++) dst = js_max(dst, fabs((double)a[i_ * n + j_])); \
  } while (0)
    double max_off;
    MAX_OFF(max_off);
    for (int64_t sweep = 0; sweep < max_sweeps && max_off > threshold; sweep++) {
      for (int64_t p = 0; p < n - 1; p++) {
        for (int64_t q = p + 1; q < n; q++) {
          const int64_t pp = p * n + p, qq = q * n + q, pq = SYM(p, q);
          const double app = a[pp], aqq = a[qq], apq = a[pq];
          if (apq == 0) continue;
          const double tau = (aqq - app) / (2 * apq);
          const double tau_sign = tau >= 0 ? 1 : -1;
          const double t = tau_sign / (fabs(tau) + sqrt(tau * tau + 1));
          const double c = 1 / sqrt(t * t + 1);
          const double s = t * c;
          for (int64_t k = 0; k < n; k++) {
            if (k == p || k == q) continue;
            const int64_t kp = SYM(k, p), kq = SYM(k, q);
            const double akp = a[kp], akq = a[kq];
            const double next_kp = c * akp - s * akq;
            const double next_kq = s * akp + c * akq;
            a[kp] = (float)next_kp;
            a[kq] = (float)next_kq;
          }
          a[pp] = (float)(c * c * app - 2 * s * c * apq + s * s * aqq);
          a[qq] = (float)(s * s * app + 2 * s * c * apq + c * c * aqq);
          a[pq] = 0;
          for (int64_t k = 0; k < n; k++) {
            const int64_t kp = k * n + p, kq = k * n + q;
            const double vkp = v[kp], vkq = v[kq];
            v[kp] = (float)(c * vkp - s * vkq);
            v[kq] = (float)(s * vkp + c * vkq);
          }
        }
      }
      MAX_OFF(max_off);
    }
#undef SYM
#undef MAX_OFF
  }
}

int ro_fft(const float* real, const float* imag, float* out_real, float* out_imag, int64_t rows, int64_t n, const int32_t* factors,
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
            const double xr = out_real[idx], xi = out_imag[idx];
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
            out_real[idx] = (float)(sum_real * stage_scale);
            out_imag[idx] = (float)(sum_imag * stage_scale);
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
