/*
 * Scalar C restatement of the attention-with-score-sums + KV-cache path of awslabs/keys_values.
 * TEST INFRASTRUCTURE ONLY: an independent second statement of oracle/kvx_oracle.py, used by the
 * tests to cross-check that module (two restatements written differently must agree) and, for the
 * quantiser, to show that the arithmetic is a fixed sequence of IEEE float32 primitives. The
 * library never links or loads it. Build: `make -C oracle` (gcc -O2 -ffp-contract=off, no
 * fast-math, so no fused multiply-add and no reassociation).
 *
 * Paths cited are relative to the reference root.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* keys_values/kvcache/quantize/pytorch.py:100-116 (scale, zero point), :120-139 (codes), one block
 * per row of D values already upcast to float32 (:333). */
void kvxo_quantize_rows(const float* x, int64_t rows, int32_t D, uint8_t* codes, float* scale, int32_t* zp) {
  for (int64_t r = 0; r < rows; ++r) {
    const float* row = x + r * (int64_t)D;
    float mn = row[0], mx = row[0];
    for (int d = 1; d < D; ++d) {
      if (row[d] < mn) mn = row[d];
      if (row[d] > mx) mx = row[d];
    }
    float s = (mx - mn) / 255.0f;
    if (s < 1.1920929e-07f) s = 1.1920929e-07f; /* clamp(min=eps) */
    int32_t z = 0 - (int32_t)rintf(mn / s);
    float inv = 1.0f / s;
    float zf = (float)z; /* float32 + int32 promotes to float32 */
    for (int d = 0; d < D; ++d) {
      float c = rintf(row[d] * inv) + zf;
      if (c < 0.0f) c = 0.0f;
      if (c > 255.0f) c = 255.0f;
      codes[r * (int64_t)D + d] = (uint8_t)c;
    }
    scale[r] = s;
    zp[r] = z;
  }
}

/* keys_values/kvcache/quantize/pytorch.py:143-154: (int32(code) - zp) converted to float32, times
 * scale. The caller rounds to the cache dtype. */
void kvxo_dequantize_rows(const uint8_t* codes, const float* scale, const int32_t* zp, int64_t rows, int32_t D,
                          float* out) {
  for (int64_t r = 0; r < rows; ++r)
    for (int d = 0; d < D; ++d) out[r * (int64_t)D + d] = (float)((int32_t)codes[r * (int64_t)D + d] - zp[r]) * scale[r];
}

/* The same quantiser with num_bits = 4 (keys_values/kvcache/quantize/pytorch.py:191-196: codes in
 * [0, 15]) and its packing, two codes per byte with the first half of the block in the high nibbles
 * (:384-393). Blocks of E float32 values (E = head_size, or n_query_groups * head_size when the
 * blocks run over the heads, :235-245); packed holds E/2 bytes per block. */
void kvxo_quantize_blocks4(const float* x, int64_t blocks, int32_t E, uint8_t* packed, float* scale, int32_t* zp) {
  uint8_t* tmp = (uint8_t*)malloc((size_t)E);
  for (int64_t r = 0; r < blocks; ++r) {
    const float* row = x + r * (int64_t)E;
    float mn = row[0], mx = row[0];
    for (int d = 1; d < E; ++d) {
      if (row[d] < mn) mn = row[d];
      if (row[d] > mx) mx = row[d];
    }
    float s = (mx - mn) / 15.0f;
    if (s < 1.1920929e-07f) s = 1.1920929e-07f;
    int32_t z = 0 - (int32_t)rintf(mn / s);
    float inv = 1.0f / s;
    float zf = (float)z;
    for (int d = 0; d < E; ++d) {
      float c = rintf(row[d] * inv) + zf;
      if (c < 0.0f) c = 0.0f;
      if (c > 15.0f) c = 15.0f;
      tmp[d] = (uint8_t)c;
    }
    for (int d = 0; d < E / 2; ++d) packed[r * (int64_t)(E / 2) + d] = (uint8_t)((tmp[d] << 4) | tmp[d + E / 2]);
    scale[r] = s;
    zp[r] = z;
  }
  free(tmp);
}

/* keys_values/kvcache/quantize/pytorch.py:457-465 (unpack: high nibbles first, then low nibbles) and
 * :143-154. */
void kvxo_dequantize_blocks4(const uint8_t* packed, const float* scale, const int32_t* zp, int64_t blocks, int32_t E,
                             float* out) {
  for (int64_t r = 0; r < blocks; ++r)
    for (int d = 0; d < E / 2; ++d) {
      uint8_t byte = packed[r * (int64_t)(E / 2) + d];
      out[r * (int64_t)E + d] = (float)((int32_t)(byte >> 4) - zp[r]) * scale[r];
      out[r * (int64_t)E + E / 2 + d] = (float)((int32_t)(byte & 15) - zp[r]) * scale[r];
    }
}

/* keys_values/attention/base.py:660-742 + keys_values/attention/attention_utils.py:383-443 as
 * explicit loops. q (B,Hq,q_len,D), k/v (B,Hkv,T,D), tp (B,Hkv,T) or NULL, all contiguous.
 * o (B,Hq,q_len,D), w (B,Hkv,T) (sum over queries, mean over the group), lse2 (B,q_len,Hq).
 * Masked pairs get the most negative float (attention_utils.py:441), as in the reference. */
void kvxo_sdpa_weights(const float* q, const float* k, const float* v, const int32_t* tp, int32_t B, int32_t Hq,
                       int32_t Hkv, int32_t q_len, int32_t T, int32_t D, int32_t input_pos, float scale, float* o,
                       float* w, float* lse2) {
  const int G = Hq / Hkv;
  float* p = (float*)malloc(sizeof(float) * (size_t)T);
  memset(w, 0, sizeof(float) * (size_t)B * Hkv * T);
  for (int b = 0; b < B; ++b)
    for (int h = 0; h < Hq; ++h) {
      const int g = h / G; /* attention_utils.py:111-122 */
      const float* kk = k + ((int64_t)b * Hkv + g) * T * D;
      const float* vv = v + ((int64_t)b * Hkv + g) * T * D;
      for (int i = 0; i < q_len; ++i) {
        const float* qq = q + (((int64_t)b * Hq + h) * q_len + i) * D;
        float m = -INFINITY;
        for (int t = 0; t < T; ++t) {
          int pos = tp ? tp[((int64_t)b * Hkv + g) * T + t] : t;
          float s;
          if (input_pos + i < pos) {
            s = -3.4028234663852886e+38f;
          } else {
            s = 0.0f;
            for (int d = 0; d < D; ++d) s += qq[d] * kk[(int64_t)t * D + d];
            s *= scale;
          }
          p[t] = s;
          if (s > m) m = s;
        }
        double z = 0.0;
        for (int t = 0; t < T; ++t) {
          p[t] = expf(p[t] - m);
          z += p[t];
        }
        float zf = (float)z;
        float* oo = o + (((int64_t)b * Hq + h) * q_len + i) * D;
        for (int d = 0; d < D; ++d) oo[d] = 0.0f;
        float* ww = w + ((int64_t)b * Hkv + g) * T;
        for (int t = 0; t < T; ++t) {
          float pt = p[t] / zf;
          ww[t] += pt / (float)G;
          for (int d = 0; d < D; ++d) oo[d] += pt * vv[(int64_t)t * D + d];
        }
        if (lse2) lse2[((int64_t)b * q_len + i) * Hq + h] = (m + logf(zf)) * 1.4426950408889634f;
      }
    }
  free(p);
}

/* keys_values/kvcache/h2o.py:175-177 (scores += w) and keys_values/kvcache/attn_weights.py:773-783
 * (the k slots with the smallest score, here in ascending (score, slot) order, by repeated linear
 * scans). scores (B,Hkv,L) contiguous, w (B,Hkv,kv_len) or NULL, next (B,Hkv,k). */
void kvxo_h2o_update_select(float* scores, const float* w, int32_t B, int32_t Hkv, int32_t L, int32_t kv_len,
                            int32_t limit, int32_t k, int32_t* next) {
  uint8_t* taken = (uint8_t*)malloc((size_t)limit);
  for (int r = 0; r < B * Hkv; ++r) {
    float* s = scores + (int64_t)r * L;
    if (w)
      for (int t = 0; t < kv_len; ++t) s[t] += w[(int64_t)r * kv_len + t];
    memset(taken, 0, (size_t)limit);
    for (int j = 0; j < k; ++j) {
      int best = -1;
      for (int t = 0; t < limit; ++t)
        if (!taken[t] && (best < 0 || s[t] < s[best])) best = t;
      taken[best] = 1;
      next[(int64_t)r * k + j] = best;
    }
  }
  free(taken);
}
