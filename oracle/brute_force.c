/*
 * Brute-force CPU attention (forward and analytic backward) in double precision.
 * TEST INFRASTRUCTURE ONLY: linked by tests, the smoke check and the benchmark's CPU-baseline leg;
 * never by the product library.
 *
 * Independent, loop-level restatement of the reference's attention for small shapes:
 *   axlearn/common/flash_attention/common.py:492-519   ReferenceMHA.__call__ (op order)
 *   axlearn/common/attention.py:2329-2380              GQA head grouping: q head n -> kv head n / G
 *   axlearn/common/attention_bias.py:43,652-658,771-790,876-882   NEG_INF and the three masks
 * Masked logits get the ADDITIVE finite bias NEG_INF per violated member mask (positional mask and
 * segment mask are separate biases that are summed, attention_bias.py:243-246).
 *
 * The backward follows the textbook softmax-attention derivative
 *   dV = P^T dO, dP = dO V^T, dS = P * (dP - rowsum(P * dP)), dQ = scale * dS K, dK = scale * dS^T Q
 * which is also what the reference's backward kernels evaluate
 * (axlearn/common/flash_attention/gpu_attention.py:507-518, 599-608).  Pinned in tests against
 * finite differences and against reverse-mode autodiff of the torch restatement.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>

#define AXL_NEG_INF (-1e15)

/* mask_kind: 0 none, 1 causal, 2 sliding-window causal (window = left context; keeps window+1). */
static double mask_bias(int mask_kind, int window, const int32_t* seg, int64_t qpos, int64_t kpos,
                        int t, int s) {
  double bias = 0.0;
  if (mask_kind == 1) {
    if (!(qpos >= kpos)) bias += AXL_NEG_INF;
  } else if (mask_kind == 2) {
    if (!((qpos >= kpos) && (qpos - kpos <= window))) bias += AXL_NEG_INF;
  }
  if (seg) {
    if (seg[t] != seg[s]) bias += AXL_NEG_INF;
  }
  return bias;
}

/*
 * q [B,T,Hq,D], k/v [B,S,Hkv,D], out [B,T,Hq,D], lse [B,Hq,T] (may be NULL), all double, dense.
 * segment_ids [B,T] int32 or NULL (requires T == S).  q_offset[b] (may be NULL) shifts the query
 * positions of batch b: position(t) = t + q_offset[b]; key positions are 0..S-1.
 */
void axl_oracle_attention_fwd(const double* q, const double* k, const double* v, double* out,
                              double* lse, const int32_t* segment_ids, const int64_t* q_offset,
                              int B, int T, int S, int Hq, int Hkv, int D, double scale,
                              int mask_kind, int window) {
  int G = Hq / Hkv;
  double* p = (double*)malloc(sizeof(double) * (size_t)S);
  for (int b = 0; b < B; b++) {
    const int32_t* seg = segment_ids ? segment_ids + (size_t)b * T : NULL;
    int64_t off = q_offset ? q_offset[b] : 0;
    for (int h = 0; h < Hq; h++) {
      int hk = h / G;
      for (int t = 0; t < T; t++) {
        const double* qr = q + (((size_t)b * T + t) * Hq + h) * D;
        double m = -INFINITY;
        for (int s = 0; s < S; s++) {
          const double* kr = k + (((size_t)b * S + s) * Hkv + hk) * D;
          double acc = 0.0;
          for (int d = 0; d < D; d++) acc += (qr[d] * scale) * kr[d];
          acc += mask_bias(mask_kind, window, seg, t + off, s, t, s);
          p[s] = acc;
          if (acc > m) m = acc;
        }
        double z = 0.0;
        for (int s = 0; s < S; s++) {
          p[s] = exp(p[s] - m);
          z += p[s];
        }
        double* orow = out + (((size_t)b * T + t) * Hq + h) * D;
        for (int d = 0; d < D; d++) orow[d] = 0.0;
        for (int s = 0; s < S; s++) {
          const double* vr = v + (((size_t)b * S + s) * Hkv + hk) * D;
          double w = p[s] / z;
          for (int d = 0; d < D; d++) orow[d] += w * vr[d];
        }
        if (lse) lse[((size_t)b * Hq + h) * T + t] = m + log(z);
      }
    }
  }
  free(p);
}

/* Gradients of sum(out * dout).  dq [B,T,Hq,D], dk/dv [B,S,Hkv,D] (summed over the G query heads). */
void axl_oracle_attention_bwd(const double* q, const double* k, const double* v, const double* dout,
                              double* dq, double* dk, double* dv, const int32_t* segment_ids,
                              const int64_t* q_offset, int B, int T, int S, int Hq, int Hkv, int D,
                              double scale, int mask_kind, int window) {
  int G = Hq / Hkv;
  double* p = (double*)malloc(sizeof(double) * (size_t)S);
  double* dp = (double*)malloc(sizeof(double) * (size_t)S);
  for (size_t i = 0; i < (size_t)B * T * Hq * D; i++) dq[i] = 0.0;
  for (size_t i = 0; i < (size_t)B * S * Hkv * D; i++) dk[i] = dv[i] = 0.0;
  for (int b = 0; b < B; b++) {
    const int32_t* seg = segment_ids ? segment_ids + (size_t)b * T : NULL;
    int64_t off = q_offset ? q_offset[b] : 0;
    for (int h = 0; h < Hq; h++) {
      int hk = h / G;
      for (int t = 0; t < T; t++) {
        const double* qr = q + (((size_t)b * T + t) * Hq + h) * D;
        const double* dor = dout + (((size_t)b * T + t) * Hq + h) * D;
        double m = -INFINITY;
        for (int s = 0; s < S; s++) {
          const double* kr = k + (((size_t)b * S + s) * Hkv + hk) * D;
          double acc = 0.0;
          for (int d = 0; d < D; d++) acc += (qr[d] * scale) * kr[d];
          acc += mask_bias(mask_kind, window, seg, t + off, s, t, s);
          p[s] = acc;
          if (acc > m) m = acc;
        }
        double z = 0.0;
        for (int s = 0; s < S; s++) {
          p[s] = exp(p[s] - m);
          z += p[s];
        }
        double delta = 0.0;
        for (int s = 0; s < S; s++) {
          const double* vr = v + (((size_t)b * S + s) * Hkv + hk) * D;
          p[s] /= z;
          double acc = 0.0;
          for (int d = 0; d < D; d++) acc += dor[d] * vr[d];
          dp[s] = acc;
          delta += p[s] * acc;
        }
        double* dqr = dq + (((size_t)b * T + t) * Hq + h) * D;
        for (int s = 0; s < S; s++) {
          const double* kr = k + (((size_t)b * S + s) * Hkv + hk) * D;
          double* dkr = dk + (((size_t)b * S + s) * Hkv + hk) * D;
          double* dvr = dv + (((size_t)b * S + s) * Hkv + hk) * D;
          double ds = p[s] * (dp[s] - delta) * scale;
          for (int d = 0; d < D; d++) {
            dqr[d] += ds * kr[d];
            dkr[d] += ds * qr[d];
            dvr[d] += p[s] * dor[d];
          }
        }
      }
    }
  }
  free(p);
  free(dp);
}

/*
 * Paged single-token decode: q [B,Hq,D]; pools [Hkv,P,page,D]; page_tables [B,pps] int32;
 * lengths [B] int32.  Token j of sequence b lives at pool[h][page_tables[b][j / page]][j % page]
 * (axlearn/common/kv_cache/paged_kv_cache.py:21-34); keys at index >= length are masked
 * (axlearn/common/flash_attention/gpu_paged_attention.py:100).  window < 0 disables the sliding
 * window; otherwise keys with (length-1) - j > window are masked as well.
 */
void axl_oracle_paged_decode(const double* q, const double* kpool, const double* vpool,
                             const int32_t* page_tables, const int32_t* lengths, double* out, int B,
                             int Hq, int Hkv, int D, int P, int page, int pps, double scale,
                             int window) {
  int G = Hq / Hkv;
  int S = pps * page;
  double* p = (double*)malloc(sizeof(double) * (size_t)S);
  for (int b = 0; b < B; b++) {
    int len = lengths[b];
    for (int h = 0; h < Hq; h++) {
      int hk = h / G;
      const double* qr = q + ((size_t)b * Hq + h) * D;
      double m = -INFINITY;
      for (int j = 0; j < S; j++) {
        int pg = page_tables[(size_t)b * pps + j / page];
        double acc = 0.0;
        if (pg >= 0 && pg < P) {
          const double* kr = kpool + (((size_t)hk * P + pg) * page + j % page) * D;
          for (int d = 0; d < D; d++) acc += (qr[d] * scale) * kr[d];
        }
        int keep = (j < len) && (window < 0 || (len - 1) - j <= window);
        if (!keep) acc += AXL_NEG_INF;
        p[j] = acc;
        if (acc > m) m = acc;
      }
      double z = 0.0;
      for (int j = 0; j < S; j++) {
        p[j] = exp(p[j] - m);
        z += p[j];
      }
      double* orow = out + ((size_t)b * Hq + h) * D;
      for (int d = 0; d < D; d++) orow[d] = 0.0;
      for (int j = 0; j < S; j++) {
        int pg = page_tables[(size_t)b * pps + j / page];
        if (!(pg >= 0 && pg < P)) continue;
        const double* vr = vpool + (((size_t)hk * P + pg) * page + j % page) * D;
        double w = p[j] / z;
        for (int d = 0; d < D; d++) orow[d] += w * vr[d];
      }
    }
  }
  free(p);
}
