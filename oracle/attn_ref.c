/*
 * CPU oracle for block-sparse attention — TEST INFRASTRUCTURE ONLY.
 *
 * This file restates, in plain C, the arithmetic the reference defines for its block-sparse attention
 * operator.  It exists to check the HIP kernels and to be timed as the CPU baseline; the product never
 * links, loads or calls it.  Only tests/, the smoke check and the benchmark's cpu_baseline leg may use it.
 *
 * Operator definition followed here (reference file:line):
 *   - allowed(i, j) = block_mask[b, h, i / q_block, j / k_block]; a 2-D mask broadcasts over (b, h):
 *     benchmark/utils/utils.py:105-119 (dense expansion), test/test_flex_block_attn.py:8-46.
 *   - O = softmax(Q K^T / sqrt(128) restricted to allowed) V, non-causal, no bias, no dropout:
 *     test/test_flex_block_attn.py:48-51 (scaled_dot_product_attention with attn_mask),
 *     flex_block_attn/flex_block_attn_h100.cu:177 (scale 1/sqrt(128)), :199-221 (online softmax), :292 (O / l).
 *   - LSE_i = log sum_j exp(s_ij) over allowed j, natural log (the kernel's "-sqrt(D)*LSE" storage form at
 *     flex_block_attn_h100.cu:303-307 is private to it and not restated).
 *   - delta_i = sum_c dO_ic O_ic: flex_block_attn_h100.cu:375-379.
 *   - P = exp(s - LSE); dV = P^T dO; dP = dO V^T; dS = P o (dP - delta) / sqrt(D); dQ = dS K; dK = dS^T Q:
 *     flex_block_attn_h100.cu:498-537, :750-753.
 *   - GQA: kv head = q head / (Hq / Hkv): flex_block_attn_h100.cu:80, :615; dK, dV sum over the q heads of a group
 *     (:555-556).
 *   - work lists: for every (b, h, i) the ascending list of selected key blocks, and for every (b, h, j) the
 *     ascending list of selecting query blocks; the reference walks the same sets by scanning the mask row
 *     (flex_block_attn_h100.cu:134-135, :247-248) or the transposed mask row (:672, :738).
 *
 * A query row with no allowed key has O = 0 and LSE = -inf here (the reference divides 0/0 there,
 * flex_block_attn_h100.cu:292; that is not reproduced).
 *
 * Accumulation is in double so that the result is a faithful fp32 reference.
 * Build: gcc -O3 -fopenmp -shared -fPIC attn_ref.c -o libattn_ref.so -lm   (oracle/build_oracle.py)
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

int oracle_num_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

void oracle_set_num_threads(int n) {
#ifdef _OPENMP
  if (n > 0) omp_set_num_threads(n);
#else
  (void)n;
#endif
}

/* mask element for (bh, I, J); mask_bh == 1 means a broadcast 2-D mask */
static inline int mask_at(const uint8_t* mask, int64_t mask_bh, int64_t bh, int nQ, int nK, int I, int J) {
  int64_t m = (mask_bh == 1) ? 0 : bh;
  return mask[(m * nQ + I) * (int64_t)nK + J] != 0;
}

/* Dense expansion of a [nQ, nK] block mask to [nQ*qbs, nK*kbs] (benchmark/utils/utils.py:105-119). */
void oracle_expand_block_mask(const uint8_t* block_mask, int nQ, int nK, int qbs, int kbs, uint8_t* dense) {
  int64_t Sk = (int64_t)nK * kbs;
  for (int I = 0; I < nQ; ++I)
    for (int r = 0; r < qbs; ++r) {
      uint8_t* row = dense + ((int64_t)I * qbs + r) * Sk;
      for (int J = 0; J < nK; ++J) memset(row + (int64_t)J * kbs, block_mask[(int64_t)I * nK + J] ? 1 : 0, (size_t)kbs);
    }
}

/*
 * Work lists.  mask: [mask_bh, nQ, nK] bytes.  q_cnt [mask_bh, nQ]; q_idx [mask_bh, nQ, nK] (first q_cnt entries
 * valid, ascending, rest -1); k_cnt [mask_bh, nK]; k_idx [mask_bh, nK, nQ] likewise.
 */
void oracle_mask_compact(const uint8_t* mask, int64_t mask_bh, int nQ, int nK, int32_t* q_cnt, int32_t* q_idx,
                         int32_t* k_cnt, int32_t* k_idx) {
  for (int64_t m = 0; m < mask_bh; ++m) {
    const uint8_t* mm = mask + m * nQ * (int64_t)nK;
    for (int I = 0; I < nQ; ++I) {
      int c = 0;
      int32_t* row = q_idx + (m * nQ + I) * (int64_t)nK;
      for (int J = 0; J < nK; ++J)
        if (mm[(int64_t)I * nK + J]) row[c++] = J;
      q_cnt[m * nQ + I] = c;
      for (; c < nK; ++c) row[c] = -1;
    }
    for (int J = 0; J < nK; ++J) {
      int c = 0;
      int32_t* row = k_idx + (m * nK + J) * (int64_t)nQ;
      for (int I = 0; I < nQ; ++I)
        if (mm[(int64_t)I * nK + J]) row[c++] = I;
      k_cnt[m * nK + J] = c;
      for (; c < nQ; ++c) row[c] = -1;
    }
  }
}

/*
 * Forward.  q [B,Hq,Sq,D], k,v [B,Hkv,Skv,D] fp32 contiguous; mask [mask_bh or 1, nQ, nK]; o [B,Hq,Sq,D]; lse [B,Hq,Sq].
 * scale = 1/sqrt(D).
 */
void oracle_attn_fwd(const float* q, const float* k, const float* v, const uint8_t* mask, int64_t mask_bh, int B, int Hq,
                     int Hkv, int Sq, int Skv, int D, int qbs, int kbs, float* o, float* lse) {
  const int nQ = Sq / qbs, nK = Skv / kbs;
  const int group = Hq / Hkv;
  const double scale = 1.0 / sqrt((double)D);
  const int64_t rows = (int64_t)B * Hq * Sq;
#pragma omp parallel
  {
    double* s = (double*)malloc(sizeof(double) * (size_t)Skv);
    double* acc = (double*)malloc(sizeof(double) * (size_t)D);
#pragma omp for schedule(dynamic, 16)
    for (int64_t r = 0; r < rows; ++r) {
      const int i = (int)(r % Sq);
      const int64_t bh = r / Sq;
      const int h = (int)(bh % Hq);
      const int b = (int)(bh / Hq);
      const int64_t kvh = (int64_t)b * Hkv + h / group;
      const float* qi = q + r * D;
      const float* kb = k + kvh * Skv * D;
      const float* vb = v + kvh * Skv * D;
      const int I = i / qbs;
      double m = -INFINITY;
      for (int J = 0; J < nK; ++J) {
        if (!mask_at(mask, mask_bh, bh, nQ, nK, I, J)) continue;
        for (int j = J * kbs; j < (J + 1) * kbs; ++j) {
          const float* kj = kb + (int64_t)j * D;
          double d = 0.0;
          for (int c = 0; c < D; ++c) d += (double)qi[c] * (double)kj[c];
          d *= scale;
          s[j] = d;
          if (d > m) m = d;
        }
      }
      for (int c = 0; c < D; ++c) acc[c] = 0.0;
      double l = 0.0;
      for (int J = 0; J < nK; ++J) {
        if (!mask_at(mask, mask_bh, bh, nQ, nK, I, J)) continue;
        for (int j = J * kbs; j < (J + 1) * kbs; ++j) {
          const double p = exp(s[j] - m);
          l += p;
          const float* vj = vb + (int64_t)j * D;
          for (int c = 0; c < D; ++c) acc[c] += p * (double)vj[c];
        }
      }
      if (l > 0.0) {
        for (int c = 0; c < D; ++c) o[r * D + c] = (float)(acc[c] / l);
        lse[r] = (float)(m + log(l));
      } else {
        for (int c = 0; c < D; ++c) o[r * D + c] = 0.0f;
        lse[r] = -INFINITY;
      }
    }
    free(s);
    free(acc);
  }
}

/* delta[r] = sum_c dO[r,c] * O[r,c]  (flex_block_attn_h100.cu:375-379) */
void oracle_bwd_delta(const float* o, const float* d_o, int64_t rows, int D, float* delta) {
#pragma omp parallel for
  for (int64_t r = 0; r < rows; ++r) {
    double a = 0.0;
    for (int c = 0; c < D; ++c) a += (double)o[r * D + c] * (double)d_o[r * D + c];
    delta[r] = (float)a;
  }
}

/*
 * Backward.  Inputs as forward plus o, lse, d_o.  Outputs dq [B,Hq,Sq,D], dk, dv [B,Hkv,Skv,D] fp32.
 * Two passes so that no accumulation races: dq is row-parallel over queries, dk/dv row-parallel over keys.
 */
void oracle_attn_bwd(const float* q, const float* k, const float* v, const float* o, const float* lse, const float* d_o,
                     const uint8_t* mask, int64_t mask_bh, int B, int Hq, int Hkv, int Sq, int Skv, int D, int qbs, int kbs,
                     float* dq, float* dk, float* dv) {
  const int nQ = Sq / qbs, nK = Skv / kbs;
  const int group = Hq / Hkv;
  const double scale = 1.0 / sqrt((double)D);
  const int64_t qrows = (int64_t)B * Hq * Sq;
  float* delta = (float*)malloc(sizeof(float) * (size_t)qrows);
  oracle_bwd_delta(o, d_o, qrows, D, delta);

  /* dQ_i = sum_j dS_ij K_j */
#pragma omp parallel
  {
    double* acc = (double*)malloc(sizeof(double) * (size_t)D);
#pragma omp for schedule(dynamic, 16)
    for (int64_t r = 0; r < qrows; ++r) {
      const int i = (int)(r % Sq);
      const int64_t bh = r / Sq;
      const int h = (int)(bh % Hq);
      const int b = (int)(bh / Hq);
      const int64_t kvh = (int64_t)b * Hkv + h / group;
      const float* qi = q + r * D;
      const float* doi = d_o + r * D;
      const float* kb = k + kvh * Skv * D;
      const float* vb = v + kvh * Skv * D;
      const int I = i / qbs;
      for (int c = 0; c < D; ++c) acc[c] = 0.0;
      for (int J = 0; J < nK; ++J) {
        if (!mask_at(mask, mask_bh, bh, nQ, nK, I, J)) continue;
        for (int j = J * kbs; j < (J + 1) * kbs; ++j) {
          const float* kj = kb + (int64_t)j * D;
          const float* vj = vb + (int64_t)j * D;
          double s = 0.0, dp = 0.0;
          for (int c = 0; c < D; ++c) {
            s += (double)qi[c] * (double)kj[c];
            dp += (double)doi[c] * (double)vj[c];
          }
          const double p = exp(s * scale - (double)lse[r]);
          const double ds = p * (dp - (double)delta[r]) * scale;
          for (int c = 0; c < D; ++c) acc[c] += ds * (double)kj[c];
        }
      }
      for (int c = 0; c < D; ++c) dq[r * D + c] = (float)acc[c];
    }
    free(acc);
  }

  /* dK_j = sum_i dS_ij Q_i ; dV_j = sum_i P_ij dO_i ; summed over the q heads of the kv head's group */
  const int64_t krows = (int64_t)B * Hkv * Skv;
#pragma omp parallel
  {
    double* ak = (double*)malloc(sizeof(double) * (size_t)D);
    double* av = (double*)malloc(sizeof(double) * (size_t)D);
#pragma omp for schedule(dynamic, 16)
    for (int64_t r = 0; r < krows; ++r) {
      const int j = (int)(r % Skv);
      const int64_t bkv = r / Skv;
      const int hk = (int)(bkv % Hkv);
      const int b = (int)(bkv / Hkv);
      const float* kj = k + r * D;
      const float* vj = v + r * D;
      const int J = j / kbs;
      for (int c = 0; c < D; ++c) ak[c] = av[c] = 0.0;
      for (int g = 0; g < group; ++g) {
        const int h = hk * group + g;
        const int64_t bh = (int64_t)b * Hq + h;
        for (int I = 0; I < nQ; ++I) {
          if (!mask_at(mask, mask_bh, bh, nQ, nK, I, J)) continue;
          for (int i = I * qbs; i < (I + 1) * qbs; ++i) {
            const int64_t qr = bh * Sq + i;
            if (!(lse[qr] > -INFINITY)) continue;
            const float* qi = q + qr * D;
            const float* doi = d_o + qr * D;
            double s = 0.0, dp = 0.0;
            for (int c = 0; c < D; ++c) {
              s += (double)qi[c] * (double)kj[c];
              dp += (double)doi[c] * (double)vj[c];
            }
            const double p = exp(s * scale - (double)lse[qr]);
            const double ds = p * (dp - (double)delta[qr]) * scale;
            for (int c = 0; c < D; ++c) {
              ak[c] += ds * (double)qi[c];
              av[c] += p * (double)doi[c];
            }
          }
        }
      }
      for (int c = 0; c < D; ++c) {
        dk[r * D + c] = (float)ak[c];
        dv[r * D + c] = (float)av[c];
      }
    }
    free(ak);
    free(av);
  }
  free(delta);
}
