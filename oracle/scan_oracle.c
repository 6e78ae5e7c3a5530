/*
 * CPU oracle for the gated linear scan -- TEST INFRASTRUCTURE, not part of the product.
 * Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may load this.
 *
 * It restates, in plain C, the sequential algorithm of the reference's CPU path:
 *   forward   quick_ssm/naive_baseline.py:28-40   h(t) = a(t)*h(t-1) + b(t)*x(t), h(-1) = 0
 *             quick_ssm/scan_interface.py:161-166 y = c*h
 *   backward  quick_ssm/naive_baseline.py:108-135 dh_total = dy*c + dh_next; dc = dy*h;
 *             db = dh_total*x; da = dh_total*h(t-1); dx = dh_total*b; dh_next = dh_total*a(t)
 * Two arithmetic flavours:
 *   *_f64      inputs are float (already rounded to their storage type by the caller), every
 *              intermediate is double: the "truth" the device results are compared with.
 *   *_f32_seq  float arithmetic in exactly the reference's operation order (one multiply, one
 *              multiply, one add per step; compile with -ffp-contract=off): bit-comparable with
 *              the torch restatement in oracle/reference_cpu_path.py for fp32 inputs.
 * All arrays are contiguous [B, L, D].  Columns (b, d) are independent, so the loops run over
 * blocks of columns in parallel and over time sequentially.
 *
 * Pinned by tests/test_oracle.py: exact rational vectors (tests/golden), closed forms, finite
 * differences, and bit-equality of the two flavours' fp32 path with the torch restatement.
 */
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define COLS 64 /* columns advanced together, for cache-friendly row access */

void oracle_scan_forward_f64(const float* x, const float* a, const float* b, const float* c, double* h,
                             double* y, int B, int L, int D) {
  const int nblk = (D + COLS - 1) / COLS;
#pragma omp parallel for collapse(2) schedule(static)
  for (int bi = 0; bi < B; ++bi) {
    for (int blk = 0; blk < nblk; ++blk) {
      const int d0 = blk * COLS, d1 = d0 + COLS < D ? d0 + COLS : D;
      double state[COLS];
      for (int k = 0; k < COLS; ++k) state[k] = 0.0;
      for (int t = 0; t < L; ++t) {
        const size_t row = ((size_t)bi * L + t) * D;
        for (int d = d0; d < d1; ++d) {
          const double s = (double)a[row + d] * state[d - d0] + (double)b[row + d] * (double)x[row + d];
          state[d - d0] = s;
          if (h) h[row + d] = s;
          if (y) y[row + d] = (c ? (double)c[row + d] : 1.0) * s;
        }
      }
    }
  }
}

/* h is rebuilt in double inside; hbuf holds one block of columns over all L. */
void oracle_scan_backward_f64(const float* x, const float* a, const float* b, const float* c, const float* dy,
                              double* dx, double* da, double* db, double* dc, int B, int L, int D) {
  const int nblk = (D + COLS - 1) / COLS;
#pragma omp parallel for collapse(2) schedule(static)
  for (int bi = 0; bi < B; ++bi) {
    for (int blk = 0; blk < nblk; ++blk) {
      const int d0 = blk * COLS, d1 = d0 + COLS < D ? d0 + COLS : D;
      double* hbuf = (double*)malloc((size_t)(L > 0 ? L : 1) * COLS * sizeof(double));
      double state[COLS], next[COLS];
      for (int k = 0; k < COLS; ++k) { state[k] = 0.0; next[k] = 0.0; }
      for (int t = 0; t < L; ++t) {
        const size_t row = ((size_t)bi * L + t) * D;
        for (int d = d0; d < d1; ++d) {
          state[d - d0] = (double)a[row + d] * state[d - d0] + (double)b[row + d] * (double)x[row + d];
          hbuf[(size_t)t * COLS + (d - d0)] = state[d - d0];
        }
      }
      for (int t = L - 1; t >= 0; --t) {
        const size_t row = ((size_t)bi * L + t) * D;
        for (int d = d0; d < d1; ++d) {
          const int k = d - d0;
          const double total = (double)dy[row + d] * (double)c[row + d] + next[k];
          const double hprev = t > 0 ? hbuf[(size_t)(t - 1) * COLS + k] : 0.0;
          dc[row + d] = (double)dy[row + d] * hbuf[(size_t)t * COLS + k];
          db[row + d] = total * (double)x[row + d];
          da[row + d] = total * hprev;
          dx[row + d] = total * (double)b[row + d];
          next[k] = total * (double)a[row + d];
        }
      }
      free(hbuf);
    }
  }
}

void oracle_scan_forward_f32_seq(const float* x, const float* a, const float* b, float* h, int B, int L, int D) {
#pragma omp parallel for schedule(static)
  for (int bi = 0; bi < B; ++bi) {
    float* state = (float*)calloc((size_t)(D > 0 ? D : 1), sizeof(float));
    for (int t = 0; t < L; ++t) {
      const size_t row = ((size_t)bi * L + t) * D;
      for (int d = 0; d < D; ++d) {
        const float decay = a[row + d] * state[d];
        const float drive = b[row + d] * x[row + d];
        state[d] = decay + drive;
        h[row + d] = state[d];
      }
    }
    free(state);
  }
}

/* fp32 in the reference's operation order; h is the forward state (as produced above). */
void oracle_scan_backward_f32_seq(const float* x, const float* a, const float* b, const float* c,
                                  const float* dy, const float* h, float* dx, float* da, float* db, float* dc,
                                  int B, int L, int D) {
#pragma omp parallel for schedule(static)
  for (int bi = 0; bi < B; ++bi) {
    float* next = (float*)calloc((size_t)(D > 0 ? D : 1), sizeof(float));
    for (int t = L - 1; t >= 0; --t) {
      const size_t row = ((size_t)bi * L + t) * D;
      for (int d = 0; d < D; ++d) {
        const float local = dy[row + d] * c[row + d];
        const float total = local + next[d];
        const float hprev = t > 0 ? h[row - D + d] : 0.0f;
        dc[row + d] = dy[row + d] * h[row + d];
        db[row + d] = total * x[row + d];
        da[row + d] = total * hprev;
        dx[row + d] = total * b[row + d];
        next[d] = total * a[row + d];
      }
    }
    free(next);
  }
}
