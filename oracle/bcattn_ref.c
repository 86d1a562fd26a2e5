/*
 * Brute-force float64 statement of block-causal attention.  TEST INFRASTRUCTURE
 * ONLY: linked by nothing in the product; loaded by tests/ (and timed by the
 * cpu_baseline leg of bench.py) to pin oracle/eager.py with an independent,
 * loop-per-element evaluation of the textbook formulas.
 *
 * Mask rule (src/opentau/policies/flash_attn_cuda/__init__.py:27-28):
 *     attend(i,j) = q_valid[i] && k_valid[j] && k_blk[j] <= q_blk[i]
 * Head map (src/opentau/policies/flash_attn_cuda/_csrc/flash_blockmask.cu:157):
 *     hk = h / (H / Hkv)
 * Rows with no visible key give O = 0, LSE = 0 and no gradient
 * (flash_blockmask.cu:240-244).
 *
 * Layout: q,o,do,dq (B,Sq,H,D); k,v,dk,dv (B,Sk,Hkv,D); lse (B,H,Sq); row-major.
 * Inputs are float32, results float64.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

static inline int attend(const int32_t *qb, const int32_t *kb, const uint8_t *qv, const uint8_t *kv,
                         int i, int j) {
  return qv[i] && kv[j] && kb[j] <= qb[i];
}

/* scores for one (b,h,i) row into s[0..Sk), returns max over visible keys; n_vis out */
static double row_scores(const float *q, const float *k, const int32_t *qb, const int32_t *kb,
                         const uint8_t *qv, const uint8_t *kv, int Sk, int Hkv, int D, int hk,
                         int i, double scale, double *s, int *n_vis) {
  double m = -INFINITY;
  int n = 0;
  for (int j = 0; j < Sk; ++j) {
    if (!attend(qb, kb, qv, kv, i, j)) {
      s[j] = -INFINITY;
      continue;
    }
    const float *kr = k + ((size_t)j * Hkv + hk) * D;
    double acc = 0.0;
    for (int d = 0; d < D; ++d) acc += (double)q[d] * (double)kr[d];
    s[j] = acc * scale;
    if (s[j] > m) m = s[j];
    ++n;
  }
  *n_vis = n;
  return m;
}

int bcref_fwd(const float *q, const float *k, const float *v, const int32_t *q_blk,
              const int32_t *k_blk, const uint8_t *q_valid, const uint8_t *k_valid, int B, int Sq,
              int Sk, int H, int Hkv, int D, double scale, double *out, double *lse) {
  if (H % Hkv) return -1;
  int G = H / Hkv;
  double *s = (double *)malloc(sizeof(double) * (size_t)Sk);
  if (!s) return -2;
  for (int b = 0; b < B; ++b) {
    const int32_t *qb = q_blk + (size_t)b * Sq, *kb = k_blk + (size_t)b * Sk;
    const uint8_t *qv = q_valid + (size_t)b * Sq, *kv = k_valid + (size_t)b * Sk;
    const float *kbase = k + (size_t)b * Sk * Hkv * D, *vbase = v + (size_t)b * Sk * Hkv * D;
    for (int h = 0; h < H; ++h) {
      int hk = h / G;
      for (int i = 0; i < Sq; ++i) {
        const float *qr = q + (((size_t)b * Sq + i) * H + h) * D;
        double *orow = out + (((size_t)b * Sq + i) * H + h) * D;
        int n;
        double m = row_scores(qr, kbase, qb, kb, qv, kv, Sk, Hkv, D, hk, i, scale, s, &n);
        memset(orow, 0, sizeof(double) * (size_t)D);
        if (n == 0) {
          lse[((size_t)b * H + h) * Sq + i] = 0.0;
          continue;
        }
        double l = 0.0;
        for (int j = 0; j < Sk; ++j)
          if (s[j] != -INFINITY) l += exp(s[j] - m);
        for (int j = 0; j < Sk; ++j) {
          if (s[j] == -INFINITY) continue;
          double p = exp(s[j] - m) / l;
          const float *vr = vbase + ((size_t)j * Hkv + hk) * D;
          for (int d = 0; d < D; ++d) orow[d] += p * (double)vr[d];
        }
        lse[((size_t)b * H + h) * Sq + i] = m + log(l);
      }
    }
  }
  free(s);
  return 0;
}

/*
 * Closed-form gradients:  P = softmax(scale*S masked),  dP = dO V^T,
 * delta_i = sum_d O_id dO_id = sum_j P_ij dP_ij,  dS = P o (dP - delta),
 * dQ = scale dS K,  dK = scale dS^T Q,  dV = P^T dO  (summed over the heads of a group).
 */
int bcref_bwd(const float *q, const float *k, const float *v, const float *dout,
              const int32_t *q_blk, const int32_t *k_blk, const uint8_t *q_valid,
              const uint8_t *k_valid, int B, int Sq, int Sk, int H, int Hkv, int D, double scale,
              double *dq, double *dk, double *dv) {
  if (H % Hkv) return -1;
  int G = H / Hkv;
  double *s = (double *)malloc(sizeof(double) * (size_t)Sk);
  double *p = (double *)malloc(sizeof(double) * (size_t)Sk);
  double *dp = (double *)malloc(sizeof(double) * (size_t)Sk);
  if (!s || !p || !dp) return -2;
  memset(dq, 0, sizeof(double) * (size_t)B * Sq * H * D);
  memset(dk, 0, sizeof(double) * (size_t)B * Sk * Hkv * D);
  memset(dv, 0, sizeof(double) * (size_t)B * Sk * Hkv * D);
  for (int b = 0; b < B; ++b) {
    const int32_t *qb = q_blk + (size_t)b * Sq, *kb = k_blk + (size_t)b * Sk;
    const uint8_t *qv = q_valid + (size_t)b * Sq, *kv = k_valid + (size_t)b * Sk;
    const float *kbase = k + (size_t)b * Sk * Hkv * D, *vbase = v + (size_t)b * Sk * Hkv * D;
    double *dkbase = dk + (size_t)b * Sk * Hkv * D, *dvbase = dv + (size_t)b * Sk * Hkv * D;
    for (int h = 0; h < H; ++h) {
      int hk = h / G;
      for (int i = 0; i < Sq; ++i) {
        size_t qoff = (((size_t)b * Sq + i) * H + h) * D;
        const float *qr = q + qoff, *dor = dout + qoff;
        double *dqr = dq + qoff;
        int n;
        double m = row_scores(qr, kbase, qb, kb, qv, kv, Sk, Hkv, D, hk, i, scale, s, &n);
        if (n == 0) continue;
        double l = 0.0;
        for (int j = 0; j < Sk; ++j)
          if (s[j] != -INFINITY) l += exp(s[j] - m);
        double delta = 0.0;
        for (int j = 0; j < Sk; ++j) {
          if (s[j] == -INFINITY) {
            p[j] = 0.0;
            dp[j] = 0.0;
            continue;
          }
          p[j] = exp(s[j] - m) / l;
          const float *vr = vbase + ((size_t)j * Hkv + hk) * D;
          double acc = 0.0;
          for (int d = 0; d < D; ++d) acc += (double)dor[d] * (double)vr[d];
          dp[j] = acc;
          delta += p[j] * acc;
        }
        for (int j = 0; j < Sk; ++j) {
          if (p[j] == 0.0 && s[j] == -INFINITY) continue;
          double ds = p[j] * (dp[j] - delta);
          const float *kr = kbase + ((size_t)j * Hkv + hk) * D;
          double *dkr = dkbase + ((size_t)j * Hkv + hk) * D;
          double *dvr = dvbase + ((size_t)j * Hkv + hk) * D;
          for (int d = 0; d < D; ++d) {
            dqr[d] += scale * ds * (double)kr[d];
            dkr[d] += scale * ds * (double)qr[d];
            dvr[d] += p[j] * (double)dor[d];
          }
        }
      }
    }
  }
  free(s);
  free(p);
  free(dp);
  return 0;
}
