/* Plain-C float64 restatement of streaming attention, forward and backward.
 *
 * TEST INFRASTRUCTURE ONLY: built into oracle/libsa_oracle.so and called from tests/
 * as an independent check of the numpy/torch oracle and of the HIP kernels.  Nothing
 * in the shipped package links or loads it.
 *
 * Semantics restated from the reference (paths relative to its repository):
 *   mask     allowed(b,i,j) = i < L_b && j < L_b && 0 <= i/C - j/C <= R,  L_b = min(lens[b], T)
 *            (src/streaming_attention/kernel.py:1540-1551, clamp at :239)
 *   forward  O_i = sum_j softmax_j(scale * q_i.k_j) v_j over allowed j; 0 for i >= L_b
 *            LSE_i = log2 sum_j exp(scale * q_i.k_j); 0 for i >= L_b           (:354-408)
 *   backward delta_i = O_i.dO_i; dP_ij = dO_i.v_j; dS_ij = P_ij (dP_ij - delta_i);
 *            dQ_i = scale sum_j dS_ij k_j; dK_j = scale sum_i dS_ij q_i; dV_j = sum_i P_ij dO_i
 *            (:1002-1022, :1105-1128)
 * Everything is a direct loop over (b, h, i, j); cost O(B H T W D).  Inputs and outputs
 * are contiguous [B,H,T,D] double arrays; lens may be NULL.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

static int64_t seq_len(const int32_t* lens, int b, int T) {
  if (!lens) return T;
  int64_t l = lens[b];
  if (l < 0) l = 0;
  return l < T ? l : T;
}

/* key range [j0, j1) that query i may attend to */
static void key_window(int64_t i, int64_t C, int64_t R, int64_t L, int64_t* j0, int64_t* j1) {
  int64_t c = i / C;
  int64_t first = c - R;
  if (first < 0) first = 0;
  *j0 = first * C;
  *j1 = (c + 1) * C < L ? (c + 1) * C : L;
}

int sa_oracle_forward(const double* q, const double* k, const double* v, const int32_t* lens,
                      double* o, double* lse, int B, int H, int T, int D, int C, int R, double scale) {
  const double log2e = 1.4426950408889634;
  double* sc = (double*)malloc(sizeof(double) * (size_t)(T > 0 ? T : 1));
  if (!sc) return -1;
  for (int b = 0; b < B; ++b) {
    const int64_t L = seq_len(lens, b, T);
    for (int h = 0; h < H; ++h) {
      const size_t base = ((size_t)b * H + h) * (size_t)T;
      for (int64_t i = 0; i < T; ++i) {
        double* oi = o + (base + i) * D;
        memset(oi, 0, sizeof(double) * D);
        lse[base + i] = 0.0;
        if (i >= L) continue;
        int64_t j0, j1;
        key_window(i, C, R, L, &j0, &j1);
        const double* qi = q + (base + i) * D;
        double mx = -INFINITY;
        for (int64_t j = j0; j < j1; ++j) {
          const double* kj = k + (base + j) * D;
          double s = 0.0;
          for (int d = 0; d < D; ++d) s += qi[d] * kj[d];
          sc[j] = s * scale;
          if (sc[j] > mx) mx = sc[j];
        }
        double den = 0.0;
        for (int64_t j = j0; j < j1; ++j) {
          sc[j] = exp(sc[j] - mx);
          den += sc[j];
        }
        for (int64_t j = j0; j < j1; ++j) {
          const double w = sc[j] / den;
          const double* vj = v + (base + j) * D;
          for (int d = 0; d < D; ++d) oi[d] += w * vj[d];
        }
        lse[base + i] = (mx + log(den)) * log2e;
      }
    }
  }
  free(sc);
  return 0;
}

/* Needs o and lse from sa_oracle_forward. dq/dk/dv are overwritten. */
int sa_oracle_backward(const double* q, const double* k, const double* v, const int32_t* lens,
                       const double* o, const double* lse, const double* d_o, double* dq, double* dk,
                       double* dv, int B, int H, int T, int D, int C, int R, double scale) {
  const double ln2 = 0.6931471805599453;
  const size_t n = (size_t)B * H * T * D;
  memset(dq, 0, sizeof(double) * n);
  memset(dk, 0, sizeof(double) * n);
  memset(dv, 0, sizeof(double) * n);
  for (int b = 0; b < B; ++b) {
    const int64_t L = seq_len(lens, b, T);
    for (int h = 0; h < H; ++h) {
      const size_t base = ((size_t)b * H + h) * (size_t)T;
      for (int64_t i = 0; i < L; ++i) {
        int64_t j0, j1;
        key_window(i, C, R, L, &j0, &j1);
        const double* qi = q + (base + i) * D;
        const double* gi = d_o + (base + i) * D;
        const double* oi = o + (base + i) * D;
        double delta = 0.0;
        for (int d = 0; d < D; ++d) delta += oi[d] * gi[d];
        for (int64_t j = j0; j < j1; ++j) {
          const double* kj = k + (base + j) * D;
          const double* vj = v + (base + j) * D;
          double s = 0.0, dp = 0.0;
          for (int d = 0; d < D; ++d) {
            s += qi[d] * kj[d];
            dp += gi[d] * vj[d];
          }
          const double p = exp(s * scale - lse[base + i] * ln2);
          const double ds = p * (dp - delta) * scale;
          double* dqi = dq + (base + i) * D;
          double* dkj = dk + (base + j) * D;
          double* dvj = dv + (base + j) * D;
          for (int d = 0; d < D; ++d) {
            dqi[d] += ds * kj[d];
            dkj[d] += ds * qi[d];
            dvj[d] += p * gi[d];
          }
        }
      }
    }
  }
  return 0;
}
