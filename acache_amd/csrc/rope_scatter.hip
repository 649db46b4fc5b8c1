// RoPE on fresh q / k rows fused with the scatter of k / v into the paged cache (gfx950).
//
// One 256-thread block per token.  A row of D elements is owned by LPR = D/2*bytes/16 lanes, each
// holding the 16 bytes at element j*VEC of the first half and the 16 bytes at the same offset of
// the second half, so the rotate-half partner (d <-> d + D/2) is in the same lane (as in the
// relocation kernel).  The block first walks the H query rows and the H_kv key rows (rotated in
// place; key rows also go to their cache slot), then copies the H_kv value rows in 16-byte chunks.
// Every row is read once; the cos / sin row of the token's position comes from L2.
#include "common.h"

// x*cos + rot_half(x)*sin with each product and the sum rounded separately, one rounding to the
// storage type: the arithmetic of the relocation kernel and of the fp32 torch formulation.
#pragma clang fp contract(off)

namespace acache {

struct RopeScatterParams {
  char *q;
  char *k;
  const char *v;
  char *k_cache;
  char *v_cache;
  const int64_t *positions;
  const int32_t *slot_map;  // NULL: no cache write
  const float *cos_tab;
  const float *sin_tab;
  int64_t N;
  int64_t num_slots;
  int64_t q_token_bytes;
  int64_t k_token_bytes;
  int64_t v_token_bytes;
  int32_t H;
  int32_t H_kv;
  int32_t rope_rows;
  int32_t D;  // head_dim (read by the any-head_dim kernel only)
};

template <int DTYPE, int D>
__global__ __launch_bounds__(256) void rope_scatter_kernel(RopeScatterParams p) {
  using E = Elem<DTYPE>;
  constexpr int VEC = E::kPerVec;
  constexpr int ROW_BYTES = D * E::kBytes;
  constexpr int HALF_BYTES = ROW_BYTES / 2;
  constexpr int LPR = HALF_BYTES / 16;  // lanes per rotated row
  constexpr int CH = ROW_BYTES / 16;    // chunks per copied row
  static_assert(HALF_BYTES % 16 == 0, "unsupported head_dim");

  const int64_t token = blockIdx.x;
  const int tid = threadIdx.x;
  const int64_t pos = p.positions[token];
  const bool rotate = pos >= 0 && pos < p.rope_rows;  // a position outside the table leaves the row unrotated
  int64_t slot = p.slot_map ? (int64_t)p.slot_map[token] : -1;
  if (slot >= p.num_slots) slot = -1;

  // this lane's table entries (the same for every row it visits)
  const int lane = tid % LPR;
  const int d0 = lane * VEC;
  float c_lo[VEC], s_lo[VEC], c_hi[VEC], s_hi[VEC];
  if (rotate) {
    const float *cr = p.cos_tab + pos * D + d0;
    const float *sr = p.sin_tab + pos * D + d0;
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
  }

  const int rows = p.H + p.H_kv;
  constexpr int RPP = 256 / LPR;  // rows per pass of the block
  for (int row = tid / LPR; row < rows; row += RPP) {
    const bool is_q = row < p.H;
    const int head = is_q ? row : row - p.H;
    char *src = is_q ? p.q + token * p.q_token_bytes : p.k + token * p.k_token_bytes;
    src += (int64_t)head * ROW_BYTES + lane * 16;
    vec16 lo = load16(src), hi = load16(src + HALF_BYTES);
    if (rotate) {
      float a[VEC], b[VEC], ya[VEC], yb[VEC];
      E::unpack(lo, a);
      E::unpack(hi, b);
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        ya[j] = a[j] * c_lo[j] + (-b[j]) * s_lo[j];
        yb[j] = b[j] * c_hi[j] + a[j] * s_hi[j];
      }
      lo = E::pack(ya);
      hi = E::pack(yb);
      store16(src, lo);
      store16(src + HALF_BYTES, hi);
    }
    if (!is_q && slot >= 0) {
      char *dst = p.k_cache + (slot * p.H_kv + head) * (int64_t)ROW_BYTES + lane * 16;
      store16(dst, lo);
      store16(dst + HALF_BYTES, hi);
    }
  }

  if (slot >= 0) {
    const char *vsrc = p.v + token * p.v_token_bytes;
    char *vdst = p.v_cache + slot * p.H_kv * (int64_t)ROW_BYTES;
    for (int c = tid; c < p.H_kv * CH; c += 256) store16(vdst + (int64_t)c * 16, load16(vsrc + (int64_t)c * 16));
  }
}

// Any other head_dim whose half row is a whole number of 16-byte chunks: the same lane layout and
// arithmetic with the row geometry in registers; a lane re-reads its table entries for every row it visits.
template <int DTYPE>
__global__ __launch_bounds__(256) void rope_scatter_any_kernel(RopeScatterParams p) {
  using E = Elem<DTYPE>;
  constexpr int VEC = E::kPerVec;
  const int D = p.D;
  const int row_bytes = D * E::kBytes;
  const int half_bytes = row_bytes / 2;
  const int lpr = half_bytes / 16;   // lanes per rotated row
  const int ch = row_bytes / 16;     // chunks per copied row

  const int64_t token = blockIdx.x;
  const int tid = threadIdx.x;
  const int64_t pos = p.positions[token];
  const bool rotate = pos >= 0 && pos < p.rope_rows;
  int64_t slot = p.slot_map ? (int64_t)p.slot_map[token] : -1;
  if (slot >= p.num_slots) slot = -1;

  const int rows = p.H + p.H_kv;
  for (int idx = tid; idx < rows * lpr; idx += 256) {
    const int row = idx / lpr, lane = idx - row * lpr;
    const bool is_q = row < p.H;
    const int head = is_q ? row : row - p.H;
    char *src = is_q ? p.q + token * p.q_token_bytes : p.k + token * p.k_token_bytes;
    src += (int64_t)head * row_bytes + lane * 16;
    vec16 lo = load16(src), hi = load16(src + half_bytes);
    if (rotate) {
      const float *cr = p.cos_tab + pos * D + lane * VEC;
      const float *sr = p.sin_tab + pos * D + lane * VEC;
      float a[VEC], b[VEC], ya[VEC], yb[VEC];
      E::unpack(lo, a);
      E::unpack(hi, b);
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        ya[j] = a[j] * cr[j] + (-b[j]) * sr[j];
        yb[j] = b[j] * cr[D / 2 + j] + a[j] * sr[D / 2 + j];
      }
      lo = E::pack(ya);
      hi = E::pack(yb);
      store16(src, lo);
      store16(src + half_bytes, hi);
    }
    if (!is_q && slot >= 0) {
      char *dst = p.k_cache + (slot * p.H_kv + head) * (int64_t)row_bytes + lane * 16;
      store16(dst, lo);
      store16(dst + half_bytes, hi);
    }
  }

  if (slot >= 0) {
    const char *vsrc = p.v + token * p.v_token_bytes;
    char *vdst = p.v_cache + slot * p.H_kv * (int64_t)row_bytes;
    for (int c = tid; c < p.H_kv * ch; c += 256) store16(vdst + (int64_t)c * 16, load16(vsrc + (int64_t)c * 16));
  }
}

template <int DTYPE, int D>
static int launch_rope_scatter(const RopeScatterParams &p, hipStream_t stream) {
  if (p.N > 0x7fffffffLL) return fail(ACACHE_E_SHAPE, "rope_qk_scatter: too many tokens (%lld)", (long long)p.N);
  hipLaunchKernelGGL((rope_scatter_kernel<DTYPE, D>), dim3((unsigned)p.N), dim3(256), 0, stream, p);
  return launch_status("rope_scatter_kernel");
}

}  // namespace acache

using namespace acache;

extern "C" int acache_rope_qk_scatter(
    void *q, void *k, const void *v, void *k_cache, void *v_cache,
    const int64_t *positions, const int32_t *slot_map, const float *rope_cos, const float *rope_sin,
    int32_t rope_rows, int64_t N, int32_t H, int32_t H_kv, int32_t D, int32_t dtype, int64_t num_slots,
    int64_t q_token_stride, int64_t k_token_stride, int64_t v_token_stride, void *stream) {
  const int es = dtype_bytes(dtype);
  if (es == 0) return fail(ACACHE_E_DTYPE, "rope_qk_scatter: unknown dtype %d", dtype);
  if (N < 0 || H <= 0 || H_kv <= 0 || num_slots < 0) return fail(ACACHE_E_SHAPE, "rope_qk_scatter: negative size");
  if (N == 0) return 0;
  if (!q || !k || !positions || !rope_cos || !rope_sin)
    return fail(ACACHE_E_NULL, "rope_qk_scatter: NULL q, k, positions or RoPE table");
  if (slot_map && (!v || !k_cache || !v_cache))
    return fail(ACACHE_E_NULL, "rope_qk_scatter: slot_map given without v or cache pointers");
  if (rope_rows <= 0) return fail(ACACHE_E_RANGE, "rope_qk_scatter: rope_rows <= 0");
  if (q_token_stride < (int64_t)H * D || k_token_stride < (int64_t)H_kv * D || (slot_map && v_token_stride < (int64_t)H_kv * D))
    return fail(ACACHE_E_SHAPE, "rope_qk_scatter: token stride smaller than one token");
  if (!aligned16(q) || !aligned16(k) || (v && !aligned16(v)) || (k_cache && !aligned16(k_cache)) ||
      (v_cache && !aligned16(v_cache)) || !aligned16(rope_cos) || !aligned16(rope_sin) ||
      (q_token_stride * es) % 16 || (k_token_stride * es) % 16 || (v_token_stride * es) % 16)
    return fail(ACACHE_E_ALIGN, "rope_qk_scatter: pointers and token strides must be 16-byte aligned");
  RopeScatterParams p;
  p.q = (char *)q; p.k = (char *)k; p.v = (const char *)v;
  p.k_cache = (char *)k_cache; p.v_cache = (char *)v_cache;
  p.positions = positions; p.slot_map = slot_map; p.cos_tab = rope_cos; p.sin_tab = rope_sin;
  p.N = N; p.num_slots = num_slots;
  p.q_token_bytes = q_token_stride * es; p.k_token_bytes = k_token_stride * es; p.v_token_bytes = v_token_stride * es;
  p.H = H; p.H_kv = H_kv; p.rope_rows = rope_rows; p.D = D;
  hipStream_t s = (hipStream_t)stream;
#define ACACHE_CASE(DT, DD) \
  if (dtype == DT && D == DD) return launch_rope_scatter<DT, DD>(p, s);
  ACACHE_CASE(ACACHE_BF16, 128)
  ACACHE_CASE(ACACHE_BF16, 64)
  ACACHE_CASE(ACACHE_F16, 128)
  ACACHE_CASE(ACACHE_F16, 64)
  ACACHE_CASE(ACACHE_F32, 128)
  ACACHE_CASE(ACACHE_F32, 64)
#undef ACACHE_CASE
  if (D <= 0 || D > 1024 || D % 2 != 0 || (D / 2 * es) % 16 != 0)
    return fail(ACACHE_E_SHAPE, "rope_qk_scatter: head_dim %d not supported (half a row must be a multiple of 16 bytes)", D);
  if (N > 0x7fffffffLL) return fail(ACACHE_E_SHAPE, "rope_qk_scatter: too many tokens (%lld)", (long long)N);
  p.D = D;
  if (dtype == ACACHE_BF16) hipLaunchKernelGGL((rope_scatter_any_kernel<ACACHE_BF16>), dim3((unsigned)N), dim3(256), 0, s, p);
  else if (dtype == ACACHE_F16) hipLaunchKernelGGL((rope_scatter_any_kernel<ACACHE_F16>), dim3((unsigned)N), dim3(256), 0, s, p);
  else hipLaunchKernelGGL((rope_scatter_any_kernel<ACACHE_F32>), dim3((unsigned)N), dim3(256), 0, s, p);
  return launch_status("rope_scatter_any_kernel");
}
