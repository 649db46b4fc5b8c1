// Affix importance for anchor selection (gfx950): for every request, the attention that its [MASK]
// queries pay to each cached affix key, soft-maxed over the affix keys only and summed over the mask
// queries and heads of one layer.
//
//   w[r, h, a]       = softmax_a( q[r, h] . rot(K[a, kv(h)], shift_b) * scale )     a in [0, A)
//   importance[b, a] += sum_{r in mask rows of b} sum_h w[r, h, a]
//
// Two launches, no atomics, so the result does not depend on scheduling:
//   1. importance_stats_kernel: one wave per (request, head, 16 mask rows) walks the affix keys and
//      leaves the row maximum and the row sum of exp (log2 domain) in the workspace;
//   2. importance_colsum_kernel: one wave per (request, 32 affix keys) walks the heads and the mask
//      rows, recomputes the scores, normalises them with the stored row statistics and accumulates
//      the column sums in registers; it is the only writer of its 32 entries of importance[b, :].
// Scores come from the matrix core (S^T = K Q^T, keys as rows, one query column per lane).  K and Q
// fragments are loaded straight from global memory in operand layout (16 bytes per lane) and the
// cached keys are re-rotated in registers; nothing goes through LDS and there is no barrier.
#include "common.h"
#include "mma.h"

namespace acache {

struct ImportanceParams {
  float *importance;
  const char *q;
  const char *k_cache;
  const int32_t *mask_rows;
  const int32_t *cu_mask;
  const int32_t *shifts;
  const float *cos_tab;
  const float *sin_tab;
  float2 *stats;
  int64_t imp_stride;
  int64_t q_token_bytes, q_head_bytes;
  int64_t kv_slot_bytes, kv_head_bytes;
  int64_t affix_slot0;
  float scale_log2e;
  int32_t A;
  int32_t B;
  int32_t H;
  int32_t H_kv;
  int32_t rope_rows;
  int32_t max_row_tiles;
};

// Operand fragments of 16 rows x D: lane (li, lg) takes row `row_ptr` (NULL: zeros), elements
// 32*ks + 8*lg .. + 8, optionally rotated by the table row (cr, sr).
template <int DTYPE, int D>
__device__ __forceinline__ void load_rows(vec16 (&f)[D / 32], const char *row_ptr, int lg, const float *cr,
                                          const float *sr) {
  constexpr int KS = D / 32;
#pragma unroll
  for (int ks = 0; ks < KS; ++ks)
    f[ks] = row_ptr ? load16(row_ptr + (32 * ks + 8 * lg) * 2) : vec16{{0, 0, 0, 0}};
  if (row_ptr && cr) {
#pragma unroll
    for (int ks = 0; ks < KS / 2; ++ks) rotate_pair<DTYPE, D>(f[ks], f[ks + KS / 2], cr, sr, 32 * ks + 8 * lg, 1.0f);
  }
}

template <int DTYPE, int D>
__global__ __launch_bounds__(256) void importance_stats_kernel(ImportanceParams p) {
  constexpr int KS = D / 32;
  using M = Mma<DTYPE>;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int li = lane & 15, lg = lane >> 4;
  const int b = blockIdx.x / p.max_row_tiles, rt = blockIdx.x % p.max_row_tiles;
  const int h = blockIdx.y * 4 + wave;
  const int m0 = p.cu_mask[b];
  const int n_rows = p.cu_mask[b + 1] - m0;
  if (h >= p.H || rt * 16 >= n_rows) return;  // no barrier in this kernel: waves may leave early
  const int kvh = h / (p.H / p.H_kv);

  const int r = rt * 16 + li;
  vec16 qf[KS];
  load_rows<DTYPE, D>(qf, r < n_rows ? p.q + (int64_t)p.mask_rows[m0 + r] * p.q_token_bytes + (int64_t)h * p.q_head_bytes
                                     : nullptr, lg, nullptr, nullptr);
  int shift = p.shifts ? p.shifts[b] : 0;
  if (shift < 0 || shift >= p.rope_rows) shift = 0;
  const float *cr = shift ? p.cos_tab + (int64_t)shift * D : nullptr;
  const float *sr = shift ? p.sin_tab + (int64_t)shift * D : nullptr;
  const char *k_base = p.k_cache + p.affix_slot0 * p.kv_slot_bytes + (int64_t)kvh * p.kv_head_bytes;
  const float c = p.scale_log2e;

  float m_run = -INFINITY, l_run = 0.0f;  // per query column (lane li); l is this lane group's share
  for (int a0 = 0; a0 < p.A; a0 += 16) {
    vec16 kf[KS];
    load_rows<DTYPE, D>(kf, a0 + li < p.A ? k_base + (int64_t)(a0 + li) * p.kv_slot_bytes : nullptr, lg, cr, sr);
    f32x4 s = {0, 0, 0, 0};
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) s = M::run(kf[ks], qf[ks], s);
    float mx = -INFINITY;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if (a0 + 4 * lg + i >= p.A) s[i] = -INFINITY;
      mx = fmaxf(mx, s[i]);
    }
    mx = fmaxf(mx, __shfl_xor(mx, 16));
    mx = fmaxf(mx, __shfl_xor(mx, 32));
    const float m_new = fmaxf(m_run, mx * c);  // finite: every tile holds at least one existing key
    float add = 0.0f;
#pragma unroll
    for (int i = 0; i < 4; ++i) add += __builtin_amdgcn_exp2f(s[i] * c - m_new);
    l_run = l_run * __builtin_amdgcn_exp2f(m_run - m_new) + add;
    m_run = m_new;
  }
  l_run += __shfl_xor(l_run, 16);
  l_run += __shfl_xor(l_run, 32);
  if (lg == 0 && r < n_rows) p.stats[(int64_t)(m0 + r) * p.H + h] = make_float2(m_run, l_run);
}

template <int DTYPE, int D>
__global__ __launch_bounds__(256) void importance_colsum_kernel(ImportanceParams p) {
  constexpr int KS = D / 32;
  constexpr int NTW = 2;  // 16-key tiles per wave
  using M = Mma<DTYPE>;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int li = lane & 15, lg = lane >> 4;
  const int b = blockIdx.y;
  const int a0 = (blockIdx.x * 4 + wave) * 16 * NTW;
  const int m0 = p.cu_mask[b];
  const int n_rows = p.cu_mask[b + 1] - m0;
  if (a0 >= p.A || n_rows <= 0) return;
  int shift = p.shifts ? p.shifts[b] : 0;
  if (shift < 0 || shift >= p.rope_rows) shift = 0;
  const float *cr = shift ? p.cos_tab + (int64_t)shift * D : nullptr;
  const float *sr = shift ? p.sin_tab + (int64_t)shift * D : nullptr;
  const float c = p.scale_log2e;
  const int group = p.H / p.H_kv;

  float col[NTW][4] = {};
  for (int h = 0; h < p.H; ++h) {
    const char *k_base = p.k_cache + p.affix_slot0 * p.kv_slot_bytes + (int64_t)(h / group) * p.kv_head_bytes;
    vec16 kf[NTW][KS];
#pragma unroll
    for (int nt = 0; nt < NTW; ++nt) {
      const int a = a0 + 16 * nt + li;
      load_rows<DTYPE, D>(kf[nt], a < p.A ? k_base + (int64_t)a * p.kv_slot_bytes : nullptr, lg, cr, sr);
    }
    for (int r0 = 0; r0 < n_rows; r0 += 16) {
      const int r = r0 + li;
      const bool live = r < n_rows;
      vec16 qf[KS];
      load_rows<DTYPE, D>(qf, live ? p.q + (int64_t)p.mask_rows[m0 + r] * p.q_token_bytes + (int64_t)h * p.q_head_bytes
                                   : nullptr, lg, nullptr, nullptr);
      const float2 st = live ? p.stats[(int64_t)(m0 + r) * p.H + h] : make_float2(0.0f, 1.0f);
      const float inv_l = live ? 1.0f / st.y : 0.0f;  // rows past the end add nothing
#pragma unroll
      for (int nt = 0; nt < NTW; ++nt) {
        f32x4 s = {0, 0, 0, 0};
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) s = M::run(kf[nt][ks], qf[ks], s);
#pragma unroll
        for (int i = 0; i < 4; ++i) col[nt][i] += __builtin_amdgcn_exp2f(s[i] * c - st.x) * inv_l;
      }
    }
  }
  // sum over the 16 query columns (lanes li) of every key row
#pragma unroll
  for (int nt = 0; nt < NTW; ++nt)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      float v = col[nt][i];
      v += __shfl_xor(v, 1);
      v += __shfl_xor(v, 2);
      v += __shfl_xor(v, 4);
      v += __shfl_xor(v, 8);
      const int a = a0 + 16 * nt + 4 * lg + i;
      if (li == 0 && a < p.A) p.importance[(int64_t)b * p.imp_stride + a] += v;
    }
}

}  // namespace acache

using namespace acache;

extern "C" int64_t acache_affix_importance_workspace_bytes(int64_t total_mask_rows, int32_t H) {
  return total_mask_rows < 0 || H < 0 ? 0 : total_mask_rows * H * (int64_t)sizeof(float2);
}

extern "C" int acache_affix_importance(
    float *importance, const void *q, const void *k_cache, const int32_t *mask_rows, const int32_t *cu_mask,
    const int32_t *affix_shifts, const float *rope_cos, const float *rope_sin, int32_t rope_rows, float scale,
    int32_t affix_len, int64_t affix_slot0, int32_t B, int64_t total_mask_rows, int32_t max_mask_rows, int32_t H,
    int32_t H_kv, int32_t D, int32_t dtype, int64_t num_slots, int64_t importance_stride, int64_t q_token_stride,
    int64_t q_head_stride, int64_t kv_slot_stride, int64_t kv_head_stride, void *workspace, int64_t workspace_bytes,
    void *stream) {
  if (dtype != ACACHE_BF16 && dtype != ACACHE_F16)
    return fail(ACACHE_E_DTYPE, "affix_importance: dtype %d not supported (bf16 or f16)", dtype);
  if (D != 128 && D != 64) return fail(ACACHE_E_SHAPE, "affix_importance: head_dim %d not supported (64 or 128)", D);
  if (B < 0 || affix_len < 0 || total_mask_rows < 0 || max_mask_rows < 0 || H <= 0 || H_kv <= 0 || H % H_kv)
    return fail(ACACHE_E_SHAPE, "affix_importance: bad sizes (B %d, A %d, H %d, H_kv %d)", B, affix_len, H, H_kv);
  if (B == 0 || affix_len == 0 || total_mask_rows == 0 || max_mask_rows == 0) return 0;
  if (!importance || !q || !k_cache || !mask_rows || !cu_mask || !workspace)
    return fail(ACACHE_E_NULL, "affix_importance: NULL pointer");
  if (affix_shifts && (!rope_cos || !rope_sin || rope_rows <= 0))
    return fail(ACACHE_E_MODE, "affix_importance: shifts given without RoPE tables");
  if (!(scale > 0.0f)) return fail(ACACHE_E_RANGE, "affix_importance: scale must be positive");
  if (affix_slot0 < 0 || affix_slot0 + affix_len > num_slots)
    return fail(ACACHE_E_RANGE, "affix_importance: affix slots [%lld, %lld) outside %lld slots", (long long)affix_slot0,
                (long long)(affix_slot0 + affix_len), (long long)num_slots);
  if (importance_stride < affix_len) return fail(ACACHE_E_SHAPE, "affix_importance: importance stride < affix_len");
  if (workspace_bytes < acache_affix_importance_workspace_bytes(total_mask_rows, H))
    return fail(ACACHE_E_SHAPE, "affix_importance: workspace of %lld bytes, %lld needed", (long long)workspace_bytes,
                (long long)acache_affix_importance_workspace_bytes(total_mask_rows, H));
  if (!aligned16(q) || !aligned16(k_cache) || !aligned16(workspace) || (rope_cos && !aligned16(rope_cos)) ||
      (rope_sin && !aligned16(rope_sin)) || (q_token_stride * 2) % 16 || (q_head_stride * 2) % 16 ||
      (kv_slot_stride * 2) % 16 || (kv_head_stride * 2) % 16)
    return fail(ACACHE_E_ALIGN, "affix_importance: pointers and strides must be 16-byte aligned");
  ImportanceParams p;
  p.importance = importance; p.q = (const char *)q; p.k_cache = (const char *)k_cache;
  p.mask_rows = mask_rows; p.cu_mask = cu_mask; p.shifts = affix_shifts;
  p.cos_tab = rope_cos; p.sin_tab = rope_sin; p.stats = (float2 *)workspace;
  p.imp_stride = importance_stride;
  p.q_token_bytes = q_token_stride * 2; p.q_head_bytes = q_head_stride * 2;
  p.kv_slot_bytes = kv_slot_stride * 2; p.kv_head_bytes = kv_head_stride * 2;
  p.affix_slot0 = affix_slot0;
  p.scale_log2e = scale * 1.4426950408889634f;
  p.A = affix_len; p.B = B; p.H = H; p.H_kv = H_kv; p.rope_rows = rope_rows;
  p.max_row_tiles = (max_mask_rows + 15) / 16;
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid1((unsigned)((int64_t)B * p.max_row_tiles), (unsigned)((H + 3) / 4));
  const dim3 grid2((unsigned)((affix_len + 127) / 128), (unsigned)B);
#define ACACHE_CASE(DT, DD)                                                                       \
  if (dtype == DT && D == DD) {                                                                   \
    hipLaunchKernelGGL((importance_stats_kernel<DT, DD>), grid1, dim3(256), 0, s, p);             \
    const int rc = launch_status("importance_stats_kernel");                                      \
    if (rc) return rc;                                                                            \
    hipLaunchKernelGGL((importance_colsum_kernel<DT, DD>), grid2, dim3(256), 0, s, p);            \
    return launch_status("importance_colsum_kernel");                                             \
  }
  ACACHE_CASE(ACACHE_BF16, 128)
  ACACHE_CASE(ACACHE_BF16, 64)
  ACACHE_CASE(ACACHE_F16, 128)
  ACACHE_CASE(ACACHE_F16, 64)
#undef ACACHE_CASE
  return fail(ACACHE_E_SHAPE, "affix_importance: unsupported dtype / head_dim");
}
