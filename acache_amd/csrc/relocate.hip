// Relocate + RoPE re-rotate + gather of cached affix K/V (gfx950).
//
// One (token, kv-head) row of D elements is owned by LPR = D/2*bytes/16 lanes.
// Lane j of a row loads the 16 bytes at element j*VEC of the FIRST half and the
// 16 bytes at the same offset of the SECOND half, so the rotate-half partner
// (d <-> d + D/2) of every element already sits in the same lane: each row is
// read from HBM exactly once and no cross-lane traffic or LDS is needed.  With
// bf16, D = 128 a wave64 covers 8 heads (2 KiB contiguous) per load pair and a
// 256-thread block covers one whole 8 KiB LLaDA token record.
//
// HBM traffic per row and layer: 2 (K,V) * 2 (read+write) * D * bytes, plus 8 B
// of slot/delta per token and the cos/sin rows, which stay in L2.
#include "common.h"

// The rotation must round each product and the sum separately (textbook
// x*cos + rot_half(x)*sin in fp32), so fused multiply-add contraction is off
// for this translation unit.
#pragma clang fp contract(off)

namespace acache {

struct RelocateParams {
  char *out_k;
  char *out_v;
  const char *k_cache;
  const char *v_cache;
  const int32_t *slot_map;  // NULL: slot = token index (in-place materialise)
  const int32_t *delta;     // NULL: const_delta for every token
  const float *cos_tab;
  const float *sin_tab;
  int64_t T;
  int64_t num_slots;
  int64_t cache_layer_bytes;
  int64_t out_layer_bytes;
  int32_t L;
  int32_t H_kv;
  int32_t rope_rows;
  int32_t const_delta;
  int32_t D;  // head_dim (read by the any-head_dim kernel only)
};

template <int DTYPE, int D, int LPB>
__global__ __launch_bounds__(256) void relocate_kernel(RelocateParams p) {
  using E = Elem<DTYPE>;
  constexpr int VEC = E::kPerVec;
  constexpr int HALF_BYTES = D / 2 * E::kBytes;
  constexpr int LPR = HALF_BYTES / 16;  // lanes per row
  constexpr int RPB = 256 / LPR;        // rows per block
  static_assert(HALF_BYTES % 16 == 0 && 256 % LPR == 0, "unsupported head_dim");

  const int tid = threadIdx.x;
  const int lane = tid % LPR;
  const int64_t row = (int64_t)blockIdx.x * RPB + tid / LPR;
  if (row >= p.T * p.H_kv) return;
  const int64_t token = row / p.H_kv;
  const int head = (int)(row - token * p.H_kv);

  const int64_t slot = p.slot_map ? (int64_t)p.slot_map[token] : token;
  const int32_t dlt = p.delta ? p.delta[token] : p.const_delta;
  const int32_t adlt = dlt < 0 ? -dlt : dlt;
  const bool rotate = dlt != 0;
  const bool valid = slot >= 0 && slot < p.num_slots && (!rotate || adlt < p.rope_rows);

  const int d0 = lane * VEC;
  float c_lo[VEC], s_lo[VEC], c_hi[VEC], s_hi[VEC];
  if (rotate && valid) {
    const float *cr = p.cos_tab + (int64_t)adlt * D + d0;
    const float *sr = p.sin_tab + (int64_t)adlt * D + d0;
#pragma unroll
    for (int j = 0; j < VEC; j += 4) {
      const float4 a = *reinterpret_cast<const float4 *>(cr + j);
      const float4 b = *reinterpret_cast<const float4 *>(sr + j);
      const float4 c = *reinterpret_cast<const float4 *>(cr + D / 2 + j);
      const float4 d = *reinterpret_cast<const float4 *>(sr + D / 2 + j);
      c_lo[j] = a.x; c_lo[j + 1] = a.y; c_lo[j + 2] = a.z; c_lo[j + 3] = a.w;
      s_lo[j] = b.x; s_lo[j + 1] = b.y; s_lo[j + 2] = b.z; s_lo[j + 3] = b.w;
      c_hi[j] = c.x; c_hi[j + 1] = c.y; c_hi[j + 2] = c.z; c_hi[j + 3] = c.w;
      s_hi[j] = d.x; s_hi[j + 1] = d.y; s_hi[j + 2] = d.z; s_hi[j + 3] = d.w;
    }
    if (dlt < 0) {  // sin is odd, cos is even: rotate by -|d|
#pragma unroll
      for (int j = 0; j < VEC; ++j) { s_lo[j] = -s_lo[j]; s_hi[j] = -s_hi[j]; }
    }
  }

  const int64_t row_bytes = (int64_t)D * E::kBytes;
  const int64_t src_off = (slot * p.H_kv + head) * row_bytes + (int64_t)lane * 16;
  const int64_t dst_off = (token * p.H_kv + head) * row_bytes + (int64_t)lane * 16;
  const int l0 = blockIdx.y * LPB;

  vec16 k_lo[LPB], k_hi[LPB], v_lo[LPB], v_hi[LPB];
  if (valid) {
#pragma unroll
    for (int i = 0; i < LPB; ++i) {
      if (l0 + i < p.L) {
        const char *ks = p.k_cache + (int64_t)(l0 + i) * p.cache_layer_bytes + src_off;
        const char *vs = p.v_cache + (int64_t)(l0 + i) * p.cache_layer_bytes + src_off;
        k_lo[i] = load16_stream(ks);
        k_hi[i] = load16_stream(ks + HALF_BYTES);
        v_lo[i] = load16_stream(vs);
        v_hi[i] = load16_stream(vs + HALF_BYTES);
      }
    }
  } else {
#pragma unroll
    for (int i = 0; i < LPB; ++i) {
      k_lo[i] = vec16{{0, 0, 0, 0}};
      k_hi[i] = k_lo[i]; v_lo[i] = k_lo[i]; v_hi[i] = k_lo[i];
    }
  }

#pragma unroll
  for (int i = 0; i < LPB; ++i) {
    if (l0 + i < p.L) {
      if (rotate && valid) {
        float a[VEC], b[VEC], ya[VEC], yb[VEC];
        E::unpack(k_lo[i], a);
        E::unpack(k_hi[i], b);
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
          // x*cos + rot_half(x)*sin with rot_half = (-x_hi, x_lo); every
          // product and the sum are rounded separately (contraction is off
          // for this file: plain operators, not the header's __f*_rn helpers,
          // whose bodies are parsed under the default contraction mode)
          ya[j] = a[j] * c_lo[j] + (-b[j]) * s_lo[j];
          yb[j] = b[j] * c_hi[j] + a[j] * s_hi[j];
        }
        k_lo[i] = E::pack(ya);
        k_hi[i] = E::pack(yb);
      }
      char *kd = p.out_k + (int64_t)(l0 + i) * p.out_layer_bytes + dst_off;
      char *vd = p.out_v + (int64_t)(l0 + i) * p.out_layer_bytes + dst_off;
      store16_writethrough(kd, k_lo[i]);
      store16_writethrough(kd + HALF_BYTES, k_hi[i]);
      store16_writethrough(vd, v_lo[i]);
      store16_writethrough(vd + HALF_BYTES, v_hi[i]);
    }
  }
}

// Any other head_dim whose half row is a whole number of 16-byte chunks (bf16 / fp16: a multiple of 16,
// fp32: a multiple of 8).  Same lane layout and the same arithmetic with the row geometry in registers
// instead of template constants: one thread per (row, chunk pair), rows packed densely into blocks.
template <int DTYPE>
__global__ __launch_bounds__(256) void relocate_any_kernel(RelocateParams p) {
  using E = Elem<DTYPE>;
  constexpr int VEC = E::kPerVec;
  const int D = p.D;
  const int half_bytes = D / 2 * E::kBytes;
  const int lpr = half_bytes / 16;

  const int64_t g = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int64_t row = g / lpr;
  const int lane = (int)(g - row * lpr);
  if (row >= p.T * p.H_kv) return;
  const int64_t token = row / p.H_kv;
  const int head = (int)(row - token * p.H_kv);

  const int64_t slot = p.slot_map ? (int64_t)p.slot_map[token] : token;
  const int32_t dlt = p.delta ? p.delta[token] : p.const_delta;
  const int32_t adlt = dlt < 0 ? -dlt : dlt;
  const bool rotate = dlt != 0;
  const bool valid = slot >= 0 && slot < p.num_slots && (!rotate || adlt < p.rope_rows);

  const int64_t row_bytes = (int64_t)D * E::kBytes;
  const int64_t src_off = (slot * p.H_kv + head) * row_bytes + (int64_t)lane * 16;
  const int64_t dst_off = (token * p.H_kv + head) * row_bytes + (int64_t)lane * 16;
  const int64_t layer = blockIdx.y;

  vec16 k_lo{{0, 0, 0, 0}}, k_hi = k_lo, v_lo = k_lo, v_hi = k_lo;
  if (valid) {
    const char *ks = p.k_cache + layer * p.cache_layer_bytes + src_off;
    const char *vs = p.v_cache + layer * p.cache_layer_bytes + src_off;
    k_lo = load16_stream(ks);
    k_hi = load16_stream(ks + half_bytes);
    v_lo = load16_stream(vs);
    v_hi = load16_stream(vs + half_bytes);
    if (rotate) {
      const int d0 = lane * VEC;
      const float *cr = p.cos_tab + (int64_t)adlt * D + d0;
      const float *sr = p.sin_tab + (int64_t)adlt * D + d0;
      const float sgn = dlt < 0 ? -1.0f : 1.0f;  // sin is odd, cos is even: rotate by -|d|
      float a[VEC], b[VEC], ya[VEC], yb[VEC];
      E::unpack(k_lo, a);
      E::unpack(k_hi, b);
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        const float cl = cr[j], sl = sgn * sr[j];
        const float ch = cr[D / 2 + j], sh = sgn * sr[D / 2 + j];
        ya[j] = a[j] * cl + (-b[j]) * sl;
        yb[j] = b[j] * ch + a[j] * sh;
      }
      k_lo = E::pack(ya);
      k_hi = E::pack(yb);
    }
  }
  char *kd = p.out_k + layer * p.out_layer_bytes + dst_off;
  char *vd = p.out_v + layer * p.out_layer_bytes + dst_off;
  store16_writethrough(kd, k_lo);
  store16_writethrough(kd + half_bytes, k_hi);
  store16_writethrough(vd, v_lo);
  store16_writethrough(vd + half_bytes, v_hi);
}

template <int DTYPE>
static int launch_relocate_any(const RelocateParams &p, hipStream_t stream) {
  const int lpr = p.D / 2 * Elem<DTYPE>::kBytes / 16;
  const int64_t threads = p.T * p.H_kv * lpr;
  if (threads == 0 || p.L == 0) return 0;
  const int64_t gx = (threads + 255) / 256;
  if (gx > 0x7fffffffLL || p.L > 65535) return fail(ACACHE_E_SHAPE, "relocate: grid too large");
  hipLaunchKernelGGL((relocate_any_kernel<DTYPE>), dim3((unsigned)gx, (unsigned)p.L), dim3(256), 0, stream, p);
  return launch_status("relocate_any_kernel");
}

template <int DTYPE, int D>
static int launch_relocate(const RelocateParams &p, hipStream_t stream) {
  constexpr int LPR = D / 2 * Elem<DTYPE>::kBytes / 16;
  constexpr int RPB = 256 / LPR;
  const int64_t rows = p.T * p.H_kv;
  if (rows == 0 || p.L == 0) return 0;
  const int64_t gx = (rows + RPB - 1) / RPB;
  if (gx > 0x7fffffffLL || p.L > 65535) return fail(ACACHE_E_SHAPE, "relocate: too many rows (%lld) or layers", (long long)rows);
  // One layer per block measured best on MI355X (5.9 TB/s against 5.4 TB/s with two
  // layers per block): the extra blocks hide more latency than deeper per-lane
  // unrolling, and token-fastest block order keeps concurrent blocks on
  // neighbouring 8 KiB records.
  constexpr int LPB = 1;
  dim3 grid((unsigned)gx, (unsigned)((p.L + LPB - 1) / LPB));
  hipLaunchKernelGGL((relocate_kernel<DTYPE, D, LPB>), grid, dim3(256), 0, stream, p);
  return launch_status("relocate_kernel");
}

static int dispatch_relocate(const RelocateParams &p, int dtype, int D, hipStream_t stream) {
#define ACACHE_CASE(DT, DD) \
  if (dtype == DT && D == DD) return launch_relocate<DT, DD>(p, stream);
  ACACHE_CASE(ACACHE_BF16, 128)
  ACACHE_CASE(ACACHE_BF16, 64)
  ACACHE_CASE(ACACHE_F16, 128)
  ACACHE_CASE(ACACHE_F16, 64)
  ACACHE_CASE(ACACHE_F32, 128)
  ACACHE_CASE(ACACHE_F32, 64)
#undef ACACHE_CASE
  const int es = dtype_bytes(dtype);
  if (es == 0) return fail(ACACHE_E_DTYPE, "relocate: unknown dtype %d", dtype);
  if (D <= 0 || D > 1024 || (D / 2 * es) % 16 != 0 || D % 2 != 0)
    return fail(ACACHE_E_SHAPE, "relocate: head_dim %d not supported (half a row must be a multiple of 16 bytes)", D);
  RelocateParams q = p;
  q.D = D;
  if (dtype == ACACHE_BF16) return launch_relocate_any<ACACHE_BF16>(q, stream);
  if (dtype == ACACHE_F16) return launch_relocate_any<ACACHE_F16>(q, stream);
  return launch_relocate_any<ACACHE_F32>(q, stream);
}

}  // namespace acache

using namespace acache;

extern "C" int acache_relocate_rope_gather(
    void *out_k, void *out_v, const void *k_cache, const void *v_cache,
    const int32_t *slot_map, const int32_t *delta, const float *rope_cos, const float *rope_sin,
    int64_t T, int32_t L, int32_t H_kv, int32_t D, int32_t dtype, int64_t num_slots,
    int32_t rope_rows, int64_t cache_layer_stride, int64_t out_layer_stride, void *stream) {
  const int es = dtype_bytes(dtype);
  if (es == 0) return fail(ACACHE_E_DTYPE, "relocate_rope_gather: unknown dtype %d", dtype);
  if (T < 0 || L < 0 || H_kv <= 0 || num_slots < 0)
    return fail(ACACHE_E_SHAPE, "relocate_rope_gather: negative size");
  if (T == 0 || L == 0) return 0;
  if (!out_k || !out_v || !k_cache || !v_cache || !slot_map)
    return fail(ACACHE_E_NULL, "relocate_rope_gather: NULL payload or slot_map pointer");
  if (delta && (!rope_cos || !rope_sin))
    return fail(ACACHE_E_MODE, "relocate_rope_gather: delta given without RoPE tables");
  if (delta && rope_rows <= 0) return fail(ACACHE_E_RANGE, "relocate_rope_gather: rope_rows <= 0");
  if (!aligned16(out_k) || !aligned16(out_v) || !aligned16(k_cache) || !aligned16(v_cache) ||
      (rope_cos && !aligned16(rope_cos)) || (rope_sin && !aligned16(rope_sin)))
    return fail(ACACHE_E_ALIGN, "relocate_rope_gather: pointers must be 16-byte aligned");
  if ((cache_layer_stride * es) % 16 || (out_layer_stride * es) % 16)
    return fail(ACACHE_E_ALIGN, "relocate_rope_gather: layer strides must be multiples of 16 bytes");
  const int64_t tok = (int64_t)H_kv * D;
  if (L > 1 && (cache_layer_stride < num_slots * tok || out_layer_stride < T * tok))
    return fail(ACACHE_E_SHAPE, "relocate_rope_gather: layer stride smaller than one layer");
  RelocateParams p;
  p.out_k = (char *)out_k; p.out_v = (char *)out_v;
  p.k_cache = (const char *)k_cache; p.v_cache = (const char *)v_cache;
  p.slot_map = slot_map; p.delta = delta; p.cos_tab = rope_cos; p.sin_tab = rope_sin;
  p.T = T; p.num_slots = num_slots;
  p.cache_layer_bytes = cache_layer_stride * es; p.out_layer_bytes = out_layer_stride * es;
  p.L = L; p.H_kv = H_kv; p.rope_rows = rope_rows; p.const_delta = 0; p.D = D;
  return dispatch_relocate(p, dtype, D, (hipStream_t)stream);
}

extern "C" int acache_materialize_relocated_affix(
    void *k_cache, void *v_cache, const float *rope_cos, const float *rope_sin,
    int64_t dst_slot, int64_t affix_len, int32_t affix_shift, int32_t L, int32_t H_kv, int32_t D,
    int32_t dtype, int64_t num_slots, int32_t rope_rows, int64_t cache_layer_stride, void *stream) {
  const int es = dtype_bytes(dtype);
  if (es == 0) return fail(ACACHE_E_DTYPE, "materialize_relocated_affix: unknown dtype %d", dtype);
  if (affix_len < 0 || L < 0 || H_kv <= 0 || num_slots < 0)
    return fail(ACACHE_E_SHAPE, "materialize_relocated_affix: negative size");
  if (affix_len == 0 || L == 0) return 0;
  if (!k_cache || !v_cache) return fail(ACACHE_E_NULL, "materialize_relocated_affix: NULL cache pointer");
  if (affix_shift != 0 && (!rope_cos || !rope_sin))
    return fail(ACACHE_E_NULL, "materialize_relocated_affix: NULL RoPE table");
  if (dst_slot < 0 || affix_len > num_slots || dst_slot > num_slots - affix_len)
    return fail(ACACHE_E_RANGE, "materialize_relocated_affix: rows [%lld, %lld) outside %lld slots",
                (long long)dst_slot, (long long)(dst_slot + affix_len), (long long)num_slots);
  if (dst_slot < affix_len)
    return fail(ACACHE_E_OVERLAP, "materialize_relocated_affix: destination %lld overlaps source [0, %lld)",
                (long long)dst_slot, (long long)affix_len);
  const int64_t ashift = affix_shift < 0 ? -(int64_t)affix_shift : affix_shift;
  if (affix_shift != 0 && ashift >= rope_rows)
    return fail(ACACHE_E_RANGE, "materialize_relocated_affix: |shift| %lld >= %d table rows",
                (long long)ashift, rope_rows);
  if (!aligned16(k_cache) || !aligned16(v_cache) || (rope_cos && !aligned16(rope_cos)) ||
      (rope_sin && !aligned16(rope_sin)) || (cache_layer_stride * es) % 16)
    return fail(ACACHE_E_ALIGN, "materialize_relocated_affix: 16-byte alignment required");
  const int64_t tok = (int64_t)H_kv * D;
  if (L > 1 && cache_layer_stride < num_slots * tok)
    return fail(ACACHE_E_SHAPE, "materialize_relocated_affix: layer stride smaller than one layer");
  RelocateParams p;
  p.out_k = (char *)k_cache + dst_slot * tok * es; p.out_v = (char *)v_cache + dst_slot * tok * es;
  p.k_cache = (const char *)k_cache; p.v_cache = (const char *)v_cache;
  p.slot_map = nullptr; p.delta = nullptr; p.cos_tab = rope_cos; p.sin_tab = rope_sin;
  p.T = affix_len; p.num_slots = num_slots;
  p.cache_layer_bytes = cache_layer_stride * es; p.out_layer_bytes = cache_layer_stride * es;
  p.L = L; p.H_kv = H_kv; p.rope_rows = rope_rows; p.const_delta = affix_shift; p.D = D;
  return dispatch_relocate(p, dtype, D, (hipStream_t)stream);
}
