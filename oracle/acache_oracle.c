/*
 * Plain-C restatement of the affix-KV reuse arithmetic.  TEST INFRASTRUCTURE ONLY:
 * linked by nothing in the product; loaded by tests/ (through oracle/c_oracle.py)
 * as a second, independent implementation that pins the torch/numpy oracle.
 *
 * Payload element types: 0 = bf16 (raw uint16), 2 = fp32.  All rotation math is
 * fp32 with every product and the sum rounded separately (compile with
 * -ffp-contract=off), one rounding to the payload type on store.
 * Citations are paths inside the reference tree.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

static float bf16_to_f32(uint16_t h) {
  uint32_t u = (uint32_t)h << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}

static uint16_t f32_to_bf16(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  if ((u & 0x7fffffffu) > 0x7f800000u) return 0x7fc0;
  return (uint16_t)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
}

static float load_elem(const void *base, int64_t i, int dtype) {
  return dtype == 0 ? bf16_to_f32(((const uint16_t *)base)[i]) : ((const float *)base)[i];
}

static void store_elem(void *base, int64_t i, int dtype, float v) {
  if (dtype == 0) ((uint16_t *)base)[i] = f32_to_bf16(v);
  else ((float *)base)[i] = v;
}

static int elem_bytes(int dtype) { return dtype == 0 ? 2 : 4; }

/* nano-vdllm/model/modeling_llada.py:392-398: inv_freq = 1/theta^(2j/D) (fp32),
 * angle = fp32(pos) * inv_freq (fp32), table = cat(angle, angle). */
void oracle_rope_table(float *cos_out, float *sin_out, int rows, int D, float theta) {
  int h = D / 2;
  for (int p = 0; p < rows; ++p)
    for (int j = 0; j < h; ++j) {
      float inv = 1.0f / powf(theta, (float)(2 * j) / (float)D);
      float ang = (float)p * inv;
      float c = cosf(ang), s = sinf(ang);
      cos_out[(int64_t)p * D + j] = c; cos_out[(int64_t)p * D + j + h] = c;
      sin_out[(int64_t)p * D + j] = s; sin_out[(int64_t)p * D + j + h] = s;
    }
}

/* One row: y = x*cos[|d|] + rot_half(x)*sgn(d)*sin[|d|]
 * (nano-vdllm/model/acache_attention.py:45-59 and 481-497). */
static void rotate_row(void *dst, const void *src, int D, int dtype, int delta,
                       const float *cos_tab, const float *sin_tab) {
  int h = D / 2, a = delta < 0 ? -delta : delta;
  const float *c = cos_tab + (int64_t)a * D, *s = sin_tab + (int64_t)a * D;
  float x[512], y[512];
  for (int d = 0; d < D; ++d) x[d] = load_elem(src, d, dtype);
  for (int d = 0; d < D; ++d) {
    float r = d < h ? -x[d + h] : x[d - h];
    float sn = delta < 0 ? -s[d] : s[d];
    float p0 = x[d] * c[d];
    float p1 = r * sn;
    y[d] = p0 + p1;
  }
  for (int d = 0; d < D; ++d) store_elem(dst, d, dtype, y[d]);
}

/* K_out[l,t] = rotate(K[l,slot[t]], delta[t]); V_out[l,t] = V[l,slot[t]].
 * Un-fused form of acache_attention.py:475-497; delta == NULL or 0 => bit copy.
 * Rows with an out-of-range slot or |delta| >= rope_rows are zero-filled. */
void oracle_relocate_rope_gather(void *out_k, void *out_v, const void *k_cache, const void *v_cache,
                                 const int32_t *slot, const int32_t *delta, const float *cos_tab,
                                 const float *sin_tab, int64_t T, int L, int H, int D, int dtype,
                                 int64_t num_slots, int rope_rows, int64_t cache_layer_stride,
                                 int64_t out_layer_stride) {
  int es = elem_bytes(dtype);
  int64_t row = (int64_t)H * D;
  for (int l = 0; l < L; ++l)
    for (int64_t t = 0; t < T; ++t) {
      char *ko = (char *)out_k + (l * out_layer_stride + t * row) * es;
      char *vo = (char *)out_v + (l * out_layer_stride + t * row) * es;
      int64_t s = slot[t];
      int d = delta ? delta[t] : 0;
      int ad = d < 0 ? -d : d;
      if (s < 0 || s >= num_slots || (d != 0 && ad >= rope_rows)) {
        memset(ko, 0, row * es);
        memset(vo, 0, row * es);
        continue;
      }
      const char *ks = (const char *)k_cache + (l * cache_layer_stride + s * row) * es;
      const char *vs = (const char *)v_cache + (l * cache_layer_stride + s * row) * es;
      memcpy(vo, vs, row * es);
      if (d == 0) { memcpy(ko, ks, row * es); continue; }
      for (int h = 0; h < H; ++h)
        rotate_row(ko + (int64_t)h * D * es, ks + (int64_t)h * D * es, D, dtype, d, cos_tab, sin_tab);
    }
}

/* cache.flat[slot[i]] = row i unless slot == -1 (nano-vdllm/model/attention.py:22-31). */
void oracle_kv_scatter(void *k_cache, void *v_cache, const void *key, const void *value,
                       const int32_t *slot, int64_t N, int H, int D, int dtype, int64_t num_slots) {
  int64_t row = (int64_t)H * D * elem_bytes(dtype);
  for (int64_t i = 0; i < N; ++i) {
    int64_t s = slot[i];
    if (s < 0 || s >= num_slots) continue;
    memcpy((char *)k_cache + s * row, (const char *)key + i * row, row);
    memcpy((char *)v_cache + s * row, (const char *)value + i * row, row);
  }
}

/* The K best of A scores, ties to the lower index, emitted ascending
 * (nano-vdllm/model_runner.py:833-843; tie rule is this build's contract).
 * Selection by repeated scan: O(A*K), for small test sizes only. */
void oracle_topk(int32_t *out, const float *scores, int A, int K, int largest) {
  char *taken = (char *)calloc((size_t)(A > 0 ? A : 1), 1);
  if (K > A) K = A;
  for (int r = 0; r < K; ++r) {
    int best = -1;
    for (int i = 0; i < A; ++i) {
      if (taken[i]) continue;
      if (best < 0) { best = i; continue; }
      float a = scores[i], b = scores[best];
      int better;
      if (isnan(a) || isnan(b)) better = largest ? (isnan(a) && !isnan(b)) : (!isnan(a) && isnan(b));
      else better = largest ? (a > b) : (a < b);
      if (better) best = i;  /* strict: an equal later index never displaces an earlier one */
    }
    taken[best] = 1;
  }
  int n = 0;
  for (int i = 0; i < A; ++i)
    if (taken[i]) out[n++] = i;
  free(taken);
}

/* out[m,h] = softmax_n(q[m,h].K[n,h/g] * scale) . V  for one request, fp32 inputs,
 * double accumulation (nano-vdllm/tests/test_attention_kernels.py:88-109). */
void oracle_dense_attention(float *out, const float *q, const float *k, const float *v, int Tq,
                            int Tk, int H, int Hkv, int D, float scale) {
  int g = H / Hkv;
  double *sc = (double *)malloc(sizeof(double) * (size_t)(Tk > 0 ? Tk : 1));
  for (int m = 0; m < Tq; ++m)
    for (int h = 0; h < H; ++h) {
      const float *qr = q + ((int64_t)m * H + h) * D;
      float *o = out + ((int64_t)m * H + h) * D;
      int kh = h / g;
      double mx = -INFINITY;
      for (int n = 0; n < Tk; ++n) {
        const float *kr = k + ((int64_t)n * Hkv + kh) * D;
        double acc = 0;
        for (int d = 0; d < D; ++d) acc += (double)qr[d] * (double)kr[d];
        sc[n] = acc * (double)scale;
        if (sc[n] > mx) mx = sc[n];
      }
      double den = 0;
      for (int n = 0; n < Tk; ++n) { sc[n] = exp(sc[n] - mx); den += sc[n]; }
      for (int d = 0; d < D; ++d) {
        double acc = 0;
        for (int n = 0; n < Tk; ++n) acc += sc[n] * (double)v[((int64_t)n * Hkv + kh) * D + d];
        o[d] = Tk > 0 ? (float)(acc / den) : 0.0f;
      }
    }
  free(sc);
}
