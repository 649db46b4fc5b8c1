// Per-request top-k anchor selection (gfx950): LDS radix select + ballot compaction.
//
// One 256-thread block per request.  Scores are mapped to order-preserving
// 32-bit keys; four 8-bit radix passes over an LDS histogram find the K-th
// largest key `thr` and how many elements equal to it are still needed.  A last
// pass walks the scores in index order and keeps every element above `thr` plus
// the first `need_eq` elements equal to it, so ties go to the lower index, and
// writes the survivors with wavefront-ballot ranks: the output is already
// ascending and no sort is needed.  Traffic: 5 reads of 4*A_b bytes (L2 hits
// after the first) and 4*K_b (or 8*K_b) bytes written per request.
#include "common.h"

namespace acache {

// Monotone map float -> uint32 (larger float => larger key).  -0 == +0; NaN is
// the largest key.  For bottom-k the key is complemented.
__device__ __forceinline__ uint32_t score_key(float x, bool largest) {
  uint32_t u;
  if (x != x) {
    u = 0xffffffffu;
  } else {
    if (x == 0.0f) x = 0.0f;  // fold -0 into +0
    u = __float_as_uint(x);
    u = (u & 0x80000000u) ? ~u : (u | 0x80000000u);
  }
  return largest ? u : ~u;
}

template <typename IdxT>
__global__ __launch_bounds__(256) void topk_kernel(
    IdxT *out, const float *scores, const int32_t *cu_affix, const int32_t *cu_k,
    const int32_t *offsets, int largest_flag) {
  __shared__ uint32_t hist[256];
  __shared__ uint32_t scan[256];
  __shared__ uint32_t sel_bin, sel_need;
  __shared__ uint32_t wave_eq[4], wave_sel[4];

  const int b = blockIdx.x;
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const bool largest = largest_flag != 0;
  const int a0 = cu_affix[b];
  const int A = cu_affix[b + 1] - a0;
  const int o0 = cu_k[b];
  const int Kreq = cu_k[b + 1] - o0;
  const int K = Kreq < A ? Kreq : (A > 0 ? A : 0);
  const int64_t add = offsets ? offsets[b] : 0;
  const float *s = scores + a0;
  IdxT *o = out + o0;

  // tail of an over-long request range: defined filler
  for (int i = K + tid; i < Kreq; i += 256) o[i] = (IdxT)-1;
  if (K <= 0) return;

  if (K == A) {  // everything is selected (the HF path short-circuits this too)
    for (int i = tid; i < A; i += 256) o[i] = (IdxT)(i + add);
    return;
  }

  // ---- radix select of the K-th largest key -------------------------------
  uint32_t prefix = 0, mask = 0, need = (uint32_t)K;
  for (int shift = 24; shift >= 0; shift -= 8) {
    hist[tid] = 0;
    __syncthreads();
    for (int i = tid; i < A; i += 256) {
      const uint32_t u = score_key(s[i], largest);
      if ((u & mask) == prefix) atomicAdd(&hist[(u >> shift) & 255u], 1u);
    }
    __syncthreads();
    // inclusive suffix sum over bins: scan[t] = sum_{bin >= t} hist[bin]
    uint32_t v = hist[tid];
    scan[tid] = v;
    __syncthreads();
    for (int step = 1; step < 256; step <<= 1) {
      const uint32_t other = (tid + step < 256) ? scan[tid + step] : 0u;
      __syncthreads();
      scan[tid] += other;
      __syncthreads();
    }
    const uint32_t incl = scan[tid];
    if (incl >= need && incl - v < need) {  // exactly one bin satisfies this
      sel_bin = (uint32_t)tid;
      sel_need = need - (incl - v);
    }
    __syncthreads();
    prefix |= sel_bin << shift;
    mask |= 255u << shift;
    need = sel_need;
    __syncthreads();
  }
  const uint32_t thr = prefix;
  const uint32_t need_eq = need;  // >= 1: how many keys == thr are kept

  // ---- ordered compaction ---------------------------------------------------
  uint32_t eq_base = 0, out_base = 0;
  for (int c0 = 0; c0 < A; c0 += 256) {
    const int i = c0 + tid;
    uint32_t u = 0;
    bool gt = false, eq = false;
    if (i < A) {
      u = score_key(s[i], largest);
      gt = u > thr;
      eq = u == thr;
    }
    const uint64_t m_eq = __ballot(eq);
    const uint64_t lt_mask = (lane == 0) ? 0ull : (~0ull >> (64 - lane));
    if (lane == 0) wave_eq[wave] = (uint32_t)__popcll(m_eq);
    __syncthreads();
    uint32_t eq_rank = eq_base + (uint32_t)__popcll(m_eq & lt_mask);
    uint32_t eq_total = 0;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      if (w < wave) eq_rank += wave_eq[w];
      eq_total += wave_eq[w];
    }
    const bool keep = gt || (eq && eq_rank < need_eq);
    const uint64_t m_keep = __ballot(keep);
    if (lane == 0) wave_sel[wave] = (uint32_t)__popcll(m_keep);
    __syncthreads();
    uint32_t pos = out_base + (uint32_t)__popcll(m_keep & lt_mask);
    uint32_t keep_total = 0;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      if (w < wave) pos += wave_sel[w];
      keep_total += wave_sel[w];
    }
    if (keep) o[pos] = (IdxT)(i + add);
    eq_base += eq_total;
    out_base += keep_total;
    __syncthreads();  // wave_eq / wave_sel are rewritten by the next chunk
  }
}

}  // namespace acache

using namespace acache;

extern "C" int acache_topk_anchors(
    void *out_idx, const float *scores, const int32_t *cu_affix, const int32_t *cu_k,
    const int32_t *offsets, int32_t largest, int32_t B, int32_t idx_bytes, void *stream) {
  if (B < 0) return fail(ACACHE_E_SHAPE, "topk_anchors: negative batch");
  if (idx_bytes != 4 && idx_bytes != 8)
    return fail(ACACHE_E_DTYPE, "topk_anchors: idx_bytes must be 4 or 8, got %d", idx_bytes);
  if (B == 0) return 0;
  if (!out_idx || !scores || !cu_affix || !cu_k) return fail(ACACHE_E_NULL, "topk_anchors: NULL pointer");
  if (idx_bytes == 4)
    hipLaunchKernelGGL(topk_kernel<int32_t>, dim3((unsigned)B), dim3(256), 0, (hipStream_t)stream,
                       (int32_t *)out_idx, scores, cu_affix, cu_k, offsets, (int)largest);
  else
    hipLaunchKernelGGL(topk_kernel<int64_t>, dim3((unsigned)B), dim3(256), 0, (hipStream_t)stream,
                       (int64_t *)out_idx, scores, cu_affix, cu_k, offsets, (int)largest);
  return launch_status("topk_kernel");
}
