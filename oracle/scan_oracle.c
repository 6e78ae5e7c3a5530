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

/* The same recurrence started from h(-1) = h0[b, d] instead of zero (h0 may be NULL), also reporting
 * h(L-1) in hfinal (may be NULL): what scanning a sequence in pieces hands from piece to piece.  The
 * reference has no such entry (its h(-1) is always zero, quick_ssm/scan_interface.py:15-21); the
 * recurrence itself is the one above.  Pinned by tests/test_oracle.py through the property that
 * pieces chained this way reproduce the whole-sequence results of the functions below. */
void oracle_scan_forward_carry_f64(const float* x, const float* a, const float* b, const float* c,
                                   const float* h0, double* h, double* y, double* hfinal, int B, int L, int D) {
  const int nblk = (D + COLS - 1) / COLS;
#pragma omp parallel for collapse(2) schedule(static)
  for (int bi = 0; bi < B; ++bi) {
    for (int blk = 0; blk < nblk; ++blk) {
      const int d0 = blk * COLS, d1 = d0 + COLS < D ? d0 + COLS : D;
      double state[COLS];
      for (int k = 0; k < COLS; ++k) state[k] = 0.0;
      if (h0) for (int d = d0; d < d1; ++d) state[d - d0] = (double)h0[(size_t)bi * D + d];
      for (int t = 0; t < L; ++t) {
        const size_t row = ((size_t)bi * L + t) * D;
        for (int d = d0; d < d1; ++d) {
          const double s = (double)a[row + d] * state[d - d0] + (double)b[row + d] * (double)x[row + d];
          state[d - d0] = s;
          if (h) h[row + d] = s;
          if (y) y[row + d] = (c ? (double)c[row + d] : 1.0) * s;
        }
      }
      if (hfinal) for (int d = d0; d < d1; ++d) hfinal[(size_t)bi * D + d] = state[d - d0];
    }
  }
}

void oracle_scan_forward_f64(const float* x, const float* a, const float* b, const float* c, double* h,
                             double* y, int B, int L, int D) {
  oracle_scan_forward_carry_f64(x, a, b, c, NULL, h, y, NULL, B, L, D);
}

/* h is rebuilt in double inside; hbuf holds one block of columns over all L. */
/* Backward of the carried-state forward: g_final[b, d] (may be NULL) is the gradient arriving at h(L-1)
 * from outside, so dh_next starts from it instead of zero; h(-1) = h0 enters da at t = 0; dh0 (may be
 * NULL) receives the gradient of h0, which is dh_next after the last (t = 0) step. */
void oracle_scan_backward_carry_f64(const float* x, const float* a, const float* b, const float* c, const float* dy,
                                    const float* h0, const float* g_final, double* dx, double* da, double* db,
                                    double* dc, double* dh0, int B, int L, int D) {
  const int nblk = (D + COLS - 1) / COLS;
#pragma omp parallel for collapse(2) schedule(static)
  for (int bi = 0; bi < B; ++bi) {
    for (int blk = 0; blk < nblk; ++blk) {
      const int d0 = blk * COLS, d1 = d0 + COLS < D ? d0 + COLS : D;
      double* hbuf = (double*)malloc((size_t)(L > 0 ? L : 1) * COLS * sizeof(double));
      double state[COLS], next[COLS];
      for (int k = 0; k < COLS; ++k) { state[k] = 0.0; next[k] = 0.0; }
      for (int d = d0; d < d1; ++d) {
        if (h0) state[d - d0] = (double)h0[(size_t)bi * D + d];
        if (g_final) next[d - d0] = (double)g_final[(size_t)bi * D + d];
      }
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
          const double hprev = t > 0 ? hbuf[(size_t)(t - 1) * COLS + k] : (h0 ? (double)h0[(size_t)bi * D + d] : 0.0);
          dc[row + d] = (double)dy[row + d] * hbuf[(size_t)t * COLS + k];
          db[row + d] = total * (double)x[row + d];
          da[row + d] = total * hprev;
          dx[row + d] = total * (double)b[row + d];
          next[k] = total * (double)a[row + d];
        }
      }
      if (dh0) for (int d = d0; d < d1; ++d) dh0[(size_t)bi * D + d] = next[d - d0];
      free(hbuf);
    }
  }
}

void oracle_scan_backward_f64(const float* x, const float* a, const float* b, const float* c, const float* dy,
                              double* dx, double* da, double* db, double* dc, int B, int L, int D) {
  oracle_scan_backward_carry_f64(x, a, b, c, dy, NULL, NULL, dx, da, db, dc, NULL, B, L, D);
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
