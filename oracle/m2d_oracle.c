/*
 * CPU oracle for the Mamba2D wavefront 2-D selective scan.
 *
 * TEST INFRASTRUCTURE ONLY.  This file is the checker the HIP kernels are
 * compared against; nothing in the shipped package may call it.  It restates,
 * in scalar C, the algorithm of the reference implementation
 * (cocoalex00/Mamba2D):
 *
 *   forward recurrence      models/kernels/wf_cuda/wf_cuda.cu:40-69
 *   output projection       models/kernels/wavefront_cuda.py:156
 *   adjoint recurrence      models/kernels/wf_cuda/wf_cuda.cu:108-160
 *   output-proj. backward   models/kernels/wavefront_cuda.py:176-178
 *   parameter gradients     models/kernels/wavefront_cuda.py:102-139
 *   d_x assembly            models/kernels/wavefront_cuda.py:193-196
 *
 * The data flow of the reference is kept on purpose (full hidden-state tensor
 * hs, in-place dBX over dHS, two-slot omega buffer indexed by row, separate
 * dDAT/dDAL tensors, masks applied afterwards), so that each intermediate can
 * be compared with an independently derived quantity in the tests.
 *
 * Layout (reference, channel-last, contiguous):
 *   x, dT, dL, y, dy : (B,H,W,E)      BT, BL, C : (B,H,W,N)
 *   AT, AL           : (E,N)          D         : (E)
 *   hs               : (B,H,W,E,N)
 *
 * Two instantiations of the same text: REAL=double (the oracle proper) and
 * REAL=float (a CPU timing baseline with the reference's fp32 arithmetic).
 *
 * Pinned by tests/test_oracle.py against: an independent pure-Python triple
 * loop, 1-D scan closed forms on the first row/column, the A=0 closed form,
 * impulse responses, linearity, transpose symmetry, and torch.autograd
 * through an independent differentiable restatement (all nine gradients and
 * the intermediates dBX, dDAT, dDAL).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

#define IDX4(b, i, j, c, H, W, C) ((((size_t)(b) * (H) + (i)) * (W) + (j)) * (size_t)(C) + (c))
#define IDX5(b, i, j, e, n, H, W, E, N) (IDX4(b, i, j, e, H, W, E) * (size_t)(N) + (n))

#define GEN(REAL, SUF, EXPF)                                                                     \
                                                                                                 \
  /* Hidden states for one batch element, all diagonals in ascending order. */                  \
  static void hs_one_batch_##SUF(int b, int H, int W, int E, int N, const REAL* x,               \
                                 const REAL* dT, const REAL* dL, const REAL* AT,                 \
                                 const REAL* AL, const REAL* BT, const REAL* BL, REAL* hs) {     \
    for (int d = 0; d < H + W - 1; ++d) {                                                        \
      int ilo = d - (W - 1) > 0 ? d - (W - 1) : 0;                                               \
      int ihi = d < H - 1 ? d : H - 1;                                                           \
      for (int i = ihi; i >= ilo; --i) {                                                         \
        int j = d - i;                                                                           \
        for (int e = 0; e < E; ++e) {                                                            \
          REAL vdt = dT[IDX4(b, i, j, e, H, W, E)];                                              \
          REAL vdl = dL[IDX4(b, i, j, e, H, W, E)];                                              \
          REAL vx = x[IDX4(b, i, j, e, H, W, E)];                                                \
          for (int n = 0; n < N; ++n) {                                                          \
            REAL gT = EXPF(vdt * AT[(size_t)e * N + n]);                                         \
            REAL gL = EXPF(vdl * AL[(size_t)e * N + n]);                                         \
            REAL uT = vdt * BT[IDX4(b, i, j, n, H, W, N)] * vx;                                  \
            REAL uL = vdl * BL[IDX4(b, i, j, n, H, W, N)] * vx;                                  \
            REAL v;                                                                              \
            if (i == 0 && j == 0) {                                                              \
              v = uL;                                                                            \
            } else if (i == 0) {                                                                 \
              v = gL * hs[IDX5(b, i, j - 1, e, n, H, W, E, N)] + uL;                             \
            } else if (j == 0) {                                                                 \
              v = gT * hs[IDX5(b, i - 1, j, e, n, H, W, E, N)] + uT;                             \
            } else {                                                                             \
              v = (REAL)0.5 * (gL * hs[IDX5(b, i, j - 1, e, n, H, W, E, N)] + uL +               \
                               gT * hs[IDX5(b, i - 1, j, e, n, H, W, E, N)] + uT);               \
            }                                                                                    \
            hs[IDX5(b, i, j, e, n, H, W, E, N)] = v;                                             \
          }                                                                                      \
        }                                                                                        \
      }                                                                                          \
    }                                                                                            \
  }                                                                                              \
                                                                                                 \
  /* hs (B,H,W,E,N) must be provided by the caller; y may be NULL. */                           \
  int m2d_oracle_fwd_##SUF(int B, int H, int W, int E, int N, const REAL* x, const REAL* dT,     \
                           const REAL* dL, const REAL* AT, const REAL* AL, const REAL* BT,       \
                           const REAL* BL, const REAL* C, const REAL* D, REAL* hs, REAL* y) {    \
    if (H < 2 || W < 2) return 1;                                                                \
    _Pragma("omp parallel for schedule(dynamic)") for (int b = 0; b < B; ++b) {                  \
      hs_one_batch_##SUF(b, H, W, E, N, x, dT, dL, AT, AL, BT, BL, hs);                          \
      if (y) {                                                                                   \
        for (int i = 0; i < H; ++i)                                                              \
          for (int j = 0; j < W; ++j)                                                            \
            for (int e = 0; e < E; ++e) {                                                        \
              REAL acc = 0;                                                                      \
              for (int n = 0; n < N; ++n)                                                        \
                acc += hs[IDX5(b, i, j, e, n, H, W, E, N)] * C[IDX4(b, i, j, n, H, W, N)];       \
              y[IDX4(b, i, j, e, H, W, E)] = acc + x[IDX4(b, i, j, e, H, W, E)] * D[e];          \
            }                                                                                    \
      }                                                                                          \
    }                                                                                            \
    return 0;                                                                                    \
  }                                                                                              \
                                                                                                 \
  /* Adjoint sweep of one batch element.  g (B,H,W,E,N) enters as dHS = dy (x) C and leaves   \
   * as dBX; omega is a (2,H,E,N) scratch for this batch element. */                            \
  static void adjoint_one_batch_##SUF(int b, int H, int W, int E, int N, const REAL* hs,         \
                                      const REAL* dT, const REAL* dL, const REAL* AT,            \
                                      const REAL* AL, REAL* g, REAL* dDAT, REAL* dDAL,           \
                                      REAL* omega) {                                             \
    size_t slot = (size_t)H * E * N;                                                             \
    for (int d = H + W - 2; d >= 0; --d) {                                                       \
      int ilo = d - (W - 1) > 0 ? d - (W - 1) : 0;                                               \
      int ihi = d < H - 1 ? d : H - 1;                                                           \
      REAL* om_next = omega + (size_t)((d + 1) & 1) * slot;                                      \
      REAL* om_curr = omega + (size_t)(d & 1) * slot;                                            \
      for (int i = ihi; i >= ilo; --i) {                                                         \
        int j = d - i;                                                                           \
        for (int e = 0; e < E; ++e)                                                              \
          for (int n = 0; n < N; ++n) {                                                          \
            REAL om_right = (j < W - 1) ? om_next[((size_t)i * E + e) * N + n] : (REAL)0;        \
            REAL om_below = (i < H - 1) ? om_next[((size_t)(i + 1) * E + e) * N + n] : (REAL)0;  \
            REAL g0 = g[IDX5(b, i, j, e, n, H, W, E, N)];                                        \
            REAL s, q;                                                                           \
            if (i == H - 1 && j == W - 1) {                                                      \
              s = g0;                                                                            \
              q = g0;                                                                            \
            } else if (i == H - 1) {                                                             \
              REAL gL = EXPF(dL[IDX4(b, i, j + 1, e, H, W, E)] * AL[(size_t)e * N + n]);         \
              q = g0 + gL * g[IDX5(b, i, j + 1, e, n, H, W, E, N)];                              \
              s = g0 + gL * om_right;                                                            \
            } else if (j == W - 1) {                                                             \
              REAL gT = EXPF(dT[IDX4(b, i + 1, j, e, H, W, E)] * AT[(size_t)e * N + n]);         \
              q = g0 + gT * g[IDX5(b, i + 1, j, e, n, H, W, E, N)];                              \
              s = g0 + gT * om_below;                                                            \
            } else {                                                                             \
              REAL gL = EXPF(dL[IDX4(b, i, j + 1, e, H, W, E)] * AL[(size_t)e * N + n]);         \
              REAL gT = EXPF(dT[IDX4(b, i + 1, j, e, H, W, E)] * AT[(size_t)e * N + n]);         \
              q = g0 + gT * g[IDX5(b, i + 1, j, e, n, H, W, E, N)] +                             \
                  gL * g[IDX5(b, i, j + 1, e, n, H, W, E, N)];                                   \
              REAL mT = (j == 0) ? (REAL)2 : (REAL)1;                                            \
              REAL mL = (i == 0) ? (REAL)2 : (REAL)1;                                            \
              s = g0 + mT * gT * om_below + mL * gL * om_right;                                  \
            }                                                                                    \
            s *= (REAL)0.5;                                                                      \
            if (i > 0 && j > 0) q *= (REAL)0.5;                                                  \
            g[IDX5(b, i, j, e, n, H, W, E, N)] = q;                                              \
            om_curr[((size_t)i * E + e) * N + n] = s;                                            \
            REAL oT = (j == 0) ? (REAL)2 : (REAL)1;                                              \
            REAL oL = (i == 0) ? (REAL)2 : (REAL)1;                                              \
            dDAT[IDX5(b, i, j, e, n, H, W, E, N)] =                                              \
                (i > 0) ? oT * s * hs[IDX5(b, i - 1, j, e, n, H, W, E, N)] : (REAL)0;            \
            dDAL[IDX5(b, i, j, e, n, H, W, E, N)] =                                              \
                (j > 0) ? oL * s * hs[IDX5(b, i, j - 1, e, n, H, W, E, N)] : (REAL)0;            \
          }                                                                                      \
      }                                                                                          \
    }                                                                                            \
  }                                                                                              \
                                                                                                 \
  /* Full backward.  Scratch tensors hs, dbx, ddat, ddal (each B*H*W*E*N) are caller-owned   \
   * and hold the reference's intermediates on return (hs, dBX, dDAT, dDAL).  d_AT, d_AL,     \
   * d_D are accumulated per batch element in ascending b order (deterministic). */           \
  int m2d_oracle_bwd_##SUF(int B, int H, int W, int E, int N, const REAL* x, const REAL* dT,     \
                           const REAL* dL, const REAL* AT, const REAL* AL, const REAL* BT,       \
                           const REAL* BL, const REAL* C, const REAL* D, const REAL* dy,         \
                           REAL* hs, REAL* dbx, REAL* ddat, REAL* ddal, REAL* d_x, REAL* d_dT,   \
                           REAL* d_dL, REAL* d_AT, REAL* d_AL, REAL* d_BT, REAL* d_BL,           \
                           REAL* d_C, REAL* d_D) {                                               \
    if (H < 2 || W < 2) return 1;                                                                \
    size_t en = (size_t)E * N;                                                                   \
    REAL* pAT = (REAL*)calloc((size_t)B * en, sizeof(REAL));                                     \
    REAL* pAL = (REAL*)calloc((size_t)B * en, sizeof(REAL));                                     \
    REAL* pD = (REAL*)calloc((size_t)B * E, sizeof(REAL));                                       \
    if (!pAT || !pAL || !pD) return 2;                                                           \
    int bad = 0;                                                                                 \
    _Pragma("omp parallel for schedule(dynamic)") for (int b = 0; b < B; ++b) {                  \
      REAL* omega = (REAL*)malloc(sizeof(REAL) * 2 * (size_t)H * en);                            \
      if (!omega) {                                                                              \
        bad = 1;                                                                                 \
        continue;                                                                                \
      }                                                                                          \
      hs_one_batch_##SUF(b, H, W, E, N, x, dT, dL, AT, AL, BT, BL, hs);                          \
      for (int i = 0; i < H; ++i)                                                                \
        for (int j = 0; j < W; ++j) {                                                            \
          for (int n = 0; n < N; ++n) d_C[IDX4(b, i, j, n, H, W, N)] = 0;                        \
          for (int e = 0; e < E; ++e) {                                                          \
            REAL gy = dy[IDX4(b, i, j, e, H, W, E)];                                             \
            pD[(size_t)b * E + e] += gy * x[IDX4(b, i, j, e, H, W, E)];                          \
            for (int n = 0; n < N; ++n) {                                                        \
              d_C[IDX4(b, i, j, n, H, W, N)] += gy * hs[IDX5(b, i, j, e, n, H, W, E, N)];        \
              dbx[IDX5(b, i, j, e, n, H, W, E, N)] = gy * C[IDX4(b, i, j, n, H, W, N)];          \
            }                                                                                    \
          }                                                                                      \
        }                                                                                        \
      adjoint_one_batch_##SUF(b, H, W, E, N, hs, dT, dL, AT, AL, dbx, ddat, ddal, omega);        \
      free(omega);                                                                               \
      for (int i = 0; i < H; ++i)                                                                \
        for (int j = 0; j < W; ++j) {                                                            \
          REAL mskT = (i > 0) ? (REAL)1 : (REAL)0;                                               \
          REAL mskL = (j > 0 || i == 0) ? (REAL)1 : (REAL)0;                                     \
          for (int n = 0; n < N; ++n) {                                                          \
            d_BT[IDX4(b, i, j, n, H, W, N)] = 0;                                                 \
            d_BL[IDX4(b, i, j, n, H, W, N)] = 0;                                                 \
          }                                                                                      \
          for (int e = 0; e < E; ++e) {                                                          \
            REAL vdt = dT[IDX4(b, i, j, e, H, W, E)];                                            \
            REAL vdl = dL[IDX4(b, i, j, e, H, W, E)];                                            \
            REAL vx = x[IDX4(b, i, j, e, H, W, E)];                                              \
            REAL a_dt = 0, a_dl = 0, a_x = 0;                                                    \
            for (int n = 0; n < N; ++n) {                                                        \
              REAL aT = AT[(size_t)e * N + n], aL = AL[(size_t)e * N + n];                       \
              REAL zT = ddat[IDX5(b, i, j, e, n, H, W, E, N)] * EXPF(vdt * aT);                  \
              REAL zL = ddal[IDX5(b, i, j, e, n, H, W, E, N)] * EXPF(vdl * aL);                  \
              pAT[(size_t)b * en + (size_t)e * N + n] += zT * vdt;                               \
              pAL[(size_t)b * en + (size_t)e * N + n] += zL * vdl;                               \
              REAL q = dbx[IDX5(b, i, j, e, n, H, W, E, N)];                                     \
              REAL qT = q * mskT, qL = q * mskL;                                                 \
              REAL bT = BT[IDX4(b, i, j, n, H, W, N)], bL = BL[IDX4(b, i, j, n, H, W, N)];       \
              a_dt += zT * aT + qT * bT * vx;                                                    \
              a_dl += zL * aL + qL * bL * vx;                                                    \
              d_BT[IDX4(b, i, j, n, H, W, N)] += qT * vdt * vx;                                  \
              d_BL[IDX4(b, i, j, n, H, W, N)] += qL * vdl * vx;                                  \
              a_x += qT * vdt * bT + qL * vdl * bL;                                              \
            }                                                                                    \
            d_dT[IDX4(b, i, j, e, H, W, E)] = a_dt;                                              \
            d_dL[IDX4(b, i, j, e, H, W, E)] = a_dl;                                              \
            d_x[IDX4(b, i, j, e, H, W, E)] = a_x + dy[IDX4(b, i, j, e, H, W, E)] * D[e];         \
          }                                                                                      \
        }                                                                                        \
    }                                                                                            \
    for (size_t k = 0; k < en; ++k) {                                                            \
      REAL sT = 0, sL = 0;                                                                       \
      for (int b = 0; b < B; ++b) {                                                              \
        sT += pAT[(size_t)b * en + k];                                                           \
        sL += pAL[(size_t)b * en + k];                                                           \
      }                                                                                          \
      d_AT[k] = sT;                                                                              \
      d_AL[k] = sL;                                                                              \
    }                                                                                            \
    for (int e = 0; e < E; ++e) {                                                                \
      REAL s = 0;                                                                                \
      for (int b = 0; b < B; ++b) s += pD[(size_t)b * E + e];                                    \
      d_D[e] = s;                                                                                \
    }                                                                                            \
    free(pAT);                                                                                   \
    free(pAL);                                                                                   \
    free(pD);                                                                                    \
    return bad ? 2 : 0;                                                                          \
  }

GEN(double, f64, exp)
GEN(float, f32, expf)

int m2d_oracle_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

void m2d_oracle_set_threads(int n) {
#ifdef _OPENMP
  if (n > 0) omp_set_num_threads(n);
#else
  (void)n;
#endif
}
