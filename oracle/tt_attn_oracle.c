/* Plain-C, double-precision restatement of triangle attention (starting node) forward and
 * backward.  TEST INFRASTRUCTURE ONLY: an independent second implementation used to pin the
 * torch oracle in tests; the shipped library never links or calls it.
 *
 * Follows the definitions implemented upstream in flash_tt_attn.py:
 *   S = sm_scale * <Q_ij, K_ik> + bias_jk           :853-857 (scale before bias), :78
 *   P = softmax_k(S), O = P V                       :860-863
 *   LSE2 = log2(sum_k exp S)                        :258
 *   delta = sum_d O*dO                              :285
 *   dP = <dO_ij, V_ik>, dS = P*(dP-delta)           :354-355, :423-424
 *   dV_ik += P dO_ij; dK_ik += sm_scale dS Q_ij     :351, :359, :518
 *   dQ_ij += sm_scale dS K_ik                       :430, :549
 *   dBias_jk += dS (summed over i, unscaled)        :426
 * All tensors are contiguous: q,k,v,o,do,dq,dk,dv (B,H,L1,L2,D); bias, dbias (B,H,L2,L2);
 * lse2 (B,H,L1,L2).  Any output pointer may be NULL.
 */
#include <math.h>
#include <stdlib.h>
#include <string.h>

int tt_attn_oracle_f64(const double* q, const double* k, const double* v, const double* bias,
                       const double* dout, double sm_scale, int B, int H, int L1, int L2, int D,
                       double* o, double* lse2, double* dq, double* dk, double* dv, double* dbias) {
  const double log2e = 1.4426950408889634;
  double* p = (double*)malloc(sizeof(double) * (size_t)L2);
  double* orow = (double*)malloc(sizeof(double) * (size_t)D);
  if (!p || !orow) { free(p); free(orow); return -1; }
  size_t nrow = (size_t)L2 * D;
  if (dq) memset(dq, 0, sizeof(double) * (size_t)B * H * L1 * nrow);
  if (dk) memset(dk, 0, sizeof(double) * (size_t)B * H * L1 * nrow);
  if (dv) memset(dv, 0, sizeof(double) * (size_t)B * H * L1 * nrow);
  if (dbias) memset(dbias, 0, sizeof(double) * (size_t)B * H * L2 * L2);
  for (int bh = 0; bh < B * H; bh++) {
    const double* bb = bias + (size_t)bh * L2 * L2;
    for (int i = 0; i < L1; i++) {
      size_t base = ((size_t)bh * L1 + i) * nrow;
      for (int j = 0; j < L2; j++) {
        const double* qj = q + base + (size_t)j * D;
        double m = -INFINITY;
        for (int kk = 0; kk < L2; kk++) {
          const double* kr = k + base + (size_t)kk * D;
          double s = 0.0;
          for (int d = 0; d < D; d++) s += qj[d] * kr[d];
          s = s * sm_scale + bb[(size_t)j * L2 + kk];
          p[kk] = s;
          if (s > m) m = s;
        }
        double z = 0.0;
        for (int kk = 0; kk < L2; kk++) { p[kk] = exp(p[kk] - m); z += p[kk]; }
        for (int kk = 0; kk < L2; kk++) p[kk] /= z;
        for (int d = 0; d < D; d++) orow[d] = 0.0;
        for (int kk = 0; kk < L2; kk++) {
          const double* vr = v + base + (size_t)kk * D;
          for (int d = 0; d < D; d++) orow[d] += p[kk] * vr[d];
        }
        if (o) memcpy(o + base + (size_t)j * D, orow, sizeof(double) * D);
        if (lse2) lse2[((size_t)bh * L1 + i) * L2 + j] = (m + log(z)) * log2e;
        if (!dout) continue;
        const double* dor = dout + base + (size_t)j * D;
        double delta = 0.0;
        for (int d = 0; d < D; d++) delta += orow[d] * dor[d];
        for (int kk = 0; kk < L2; kk++) {
          const double* vr = v + base + (size_t)kk * D;
          const double* kr = k + base + (size_t)kk * D;
          double dp = 0.0;
          for (int d = 0; d < D; d++) dp += dor[d] * vr[d];
          double ds = p[kk] * (dp - delta);
          if (dbias) dbias[((size_t)bh * L2 + j) * L2 + kk] += ds;
          for (int d = 0; d < D; d++) {
            if (dv) dv[base + (size_t)kk * D + d] += p[kk] * dor[d];
            if (dk) dk[base + (size_t)kk * D + d] += sm_scale * ds * qj[d];
            if (dq) dq[base + (size_t)j * D + d] += sm_scale * ds * kr[d];
          }
        }
      }
    }
  }
  free(p); free(orow);
  return 0;
}
