// Token proposal and its confidence for masked-diffusion decoding (gfx950): per logits row the arg-max
// token and exp(logit[token] - logsumexp(row)), in one streaming pass over the vocabulary.
//
// One 1024-thread block per row.  A thread walks 16-byte chunks of the row (stride 1024 chunks, four loads
// in flight) keeping an online (max, first index of the max, sum of exp(x - max)) triple in fp32; the
// triples are merged across the wave with shuffles and across the sixteen waves through LDS.  The row is
// read once (the torch formulation up-casts it to fp32, gathers, and reduces it twice); bound: HBM,
// V * bytes per row.
#include "common.h"

namespace acache {

struct ConfidenceParams {
  int64_t *out_token;   // may be NULL when picks are given
  float *out_conf;
  const char *logits;
  const int64_t *picks;  // NULL: confidence of the arg-max token
  int64_t V;
  int64_t row_bytes;
};

template <int DTYPE>
__device__ __forceinline__ float load_elem(const char *p) {
  if (DTYPE == ACACHE_F32) return *reinterpret_cast<const float *>(p);
  const uint32_t h = *reinterpret_cast<const uint16_t *>(p);
  return DTYPE == ACACHE_BF16 ? bf16_to_f32(h) : f16_to_f32(h);
}

struct RowStat {
  float m;      // running maximum
  float s;      // sum of exp(x - m)
  int64_t idx;  // first index holding m
};

__device__ __forceinline__ RowStat merge(const RowStat &a, const RowStat &b) {
  RowStat r;
  r.m = fmaxf(a.m, b.m);
  const float sa = a.m == -INFINITY ? 0.0f : a.s * __expf(a.m - r.m);
  const float sb = b.m == -INFINITY ? 0.0f : b.s * __expf(b.m - r.m);
  r.s = sa + sb;
  r.idx = a.m > b.m ? a.idx : (b.m > a.m ? b.idx : (a.idx < b.idx ? a.idx : b.idx));
  return r;
}

constexpr int kConfThreads = 1024;

template <int DTYPE>
__global__ __launch_bounds__(kConfThreads) void confidence_kernel(ConfidenceParams p) {
  using E = Elem<DTYPE>;
  constexpr int VEC = E::kPerVec;
  const int tid = threadIdx.x;
  const char *row = p.logits + (int64_t)blockIdx.x * p.row_bytes;

  RowStat st{-INFINITY, 0.0f, INT64_MAX};
  auto take = [&](const float (&x)[VEC], int n, int64_t base) {
    float cm = -INFINITY;
    for (int j = 0; j < n; ++j) cm = fmaxf(cm, x[j]);  // NaN never wins: fmaxf returns the other operand
    if (cm == -INFINITY) return;             // nothing finite here: contributes zero
    if (cm > st.m) {                         // rare after the first chunks: only then look for the position
      int ci = 0;
      for (int j = n - 1; j >= 0; --j)
        if (x[j] == cm) ci = j;              // the first maximum wins
      st.s *= __expf(st.m - cm);             // exp(-inf) = 0 on the first chunk
      st.m = cm;
      st.idx = base + ci;
    }
    float add = 0.0f;
    for (int j = 0; j < n; ++j) add += __expf(x[j] - st.m);
    st.s += add;
  };

  const int64_t full = p.V / VEC;
  int64_t c = tid;
  constexpr int kInFlight = 4;  // independent loads before any use (8 measured no better)
  for (; c + (kInFlight - 1) * kConfThreads < full; c += kInFlight * kConfThreads) {
    vec16 raw[kInFlight];
#pragma unroll
    for (int u = 0; u < kInFlight; ++u) raw[u] = load16_stream(row + (c + u * kConfThreads) * 16);
#pragma unroll
    for (int u = 0; u < kInFlight; ++u) {
      float x[VEC];
      E::unpack(raw[u], x);
      take(x, VEC, (c + u * kConfThreads) * VEC);
    }
  }
  for (; c < full; c += kConfThreads) {
    float x[VEC];
    E::unpack(load16_stream(row + c * 16), x);
    take(x, VEC, c * VEC);
  }
  if (tid == 0 && full * VEC < p.V) {  // ragged tail of the vocabulary, element by element
    float x[VEC];
    const int n = (int)(p.V - full * VEC);
    for (int j = 0; j < VEC; ++j) x[j] = j < n ? load_elem<DTYPE>(row + (full * VEC + j) * E::kBytes) : -INFINITY;
    take(x, n, full * VEC);
  }

#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) {
    RowStat o;
    o.m = __shfl_xor(st.m, d);
    o.s = __shfl_xor(st.s, d);
    o.idx = __shfl_xor((long long)st.idx, d);
    st = merge(st, o);
  }
  constexpr int WAVES = kConfThreads / 64;
  __shared__ float sm[WAVES], ss[WAVES];
  __shared__ long long si[WAVES];
  if ((tid & 63) == 0) { sm[tid >> 6] = st.m; ss[tid >> 6] = st.s; si[tid >> 6] = st.idx; }
  __syncthreads();
  if (tid == 0) {
    RowStat r{sm[0], ss[0], si[0]};
    for (int w = 1; w < WAVES; ++w) r = merge(r, RowStat{sm[w], ss[w], si[w]});
    float chosen = r.m;
    if (p.picks) {
      const int64_t pick = p.picks[blockIdx.x];
      chosen = pick >= 0 && pick < p.V ? load_elem<DTYPE>(row + pick * E::kBytes) : -INFINITY;
    } else if (r.idx == INT64_MAX) {
      r.idx = 0;  // a row of -inf: torch.argmax answers 0
    }
    if (p.out_token) p.out_token[blockIdx.x] = p.picks ? p.picks[blockIdx.x] : r.idx;
    p.out_conf[blockIdx.x] = expf(chosen - (r.m + logf(r.s)));
  }
}

}  // namespace acache

using namespace acache;

// The commit rule of block-wise decoding on one row of a block per wave: among the positions that still hold the
// mask token and whose proposal is another token, commit the proposals whose confidence reaches the threshold, and
// when there are such positions but none reaches it, the most confident one (the first of equals).  Positions are
// walked twice (decide, then write); a row is 32 to a few hundred positions.
__global__ __launch_bounds__(64) void commit_tokens_kernel(int64_t *blocks, const int64_t *proposal, const float *conf,
                                                           int32_t *committed_rows, int L, int64_t mask_id,
                                                           float threshold) {
  const int lane = threadIdx.x;
  int64_t *row = blocks + (int64_t)blockIdx.x * L;
  const int64_t *prop = proposal + (int64_t)blockIdx.x * L;
  const float *cf = conf + (int64_t)blockIdx.x * L;
  bool any_committable = false, any_above = false;
  float best = -INFINITY;
  int best_at = 0x7fffffff;
  for (int i = lane; i < L; i += 64) {
    const bool committable = row[i] == mask_id && prop[i] != mask_id;
    if (!committable) continue;
    const float c = cf[i];
    any_committable = true;
    any_above |= c >= threshold;
    if (c > best || best_at == 0x7fffffff) { best = c; best_at = i; }  // i ascends: the first of equals stays
  }
  const bool row_committable = __builtin_amdgcn_ballot_w64(any_committable) != 0;
  const bool row_above = __builtin_amdgcn_ballot_w64(any_above) != 0;
  if (!row_committable) return;
  int forced = -1;
  if (!row_above) {
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) {
      const float ob = __shfl_xor(best, d);
      const int oa = __shfl_xor(best_at, d);
      if (oa != 0x7fffffff && (best_at == 0x7fffffff || ob > best || (ob == best && oa < best_at))) { best = ob; best_at = oa; }
    }
    forced = best_at;
  }
  for (int i = lane; i < L; i += 64) {
    const int64_t tok = prop[i];
    const bool committable = row[i] == mask_id && tok != mask_id;
    if (committable && (i == forced || (row_above && cf[i] >= threshold))) row[i] = tok;
  }
  if (lane == 0) atomicAdd(committed_rows, 1);
}

extern "C" int acache_commit_tokens(int64_t *blocks, const int64_t *proposal, const float *confidence,
                                    int32_t *committed_rows, int64_t n, int32_t L, int64_t mask_id, float threshold,
                                    void *stream) {
  if (n < 0 || L <= 0) return fail(ACACHE_E_SHAPE, "commit_tokens: n %lld, L %d", (long long)n, L);
  if (n == 0) return 0;
  if (!blocks || !proposal || !confidence || !committed_rows) return fail(ACACHE_E_NULL, "commit_tokens: NULL pointer");
  if (n > 0x7fffffffLL) return fail(ACACHE_E_SHAPE, "commit_tokens: too many rows");
  hipLaunchKernelGGL(commit_tokens_kernel, dim3((unsigned)n), dim3(64), 0, (hipStream_t)stream, blocks, proposal,
                     confidence, committed_rows, L, mask_id, threshold);
  return launch_status("commit_tokens_kernel");
}

extern "C" int acache_argmax_confidence(
    int64_t *out_token, float *out_conf, const void *logits, const int64_t *picks,
    int64_t R, int64_t V, int64_t row_stride, int32_t dtype, void *stream) {
  const int es = dtype_bytes(dtype);
  if (es == 0) return fail(ACACHE_E_DTYPE, "argmax_confidence: unknown dtype %d", dtype);
  if (R < 0 || V <= 0) return fail(ACACHE_E_SHAPE, "argmax_confidence: R %lld, V %lld", (long long)R, (long long)V);
  if (R == 0) return 0;
  if (!out_conf || !logits || (!out_token && !picks))
    return fail(ACACHE_E_NULL, "argmax_confidence: NULL output or logits pointer");
  if (row_stride < V) return fail(ACACHE_E_SHAPE, "argmax_confidence: row stride %lld < V %lld", (long long)row_stride, (long long)V);
  if (!aligned16(logits) || (row_stride * es) % 16)
    return fail(ACACHE_E_ALIGN, "argmax_confidence: logits and the row stride must be 16-byte aligned");
  if (R > 0x7fffffffLL) return fail(ACACHE_E_SHAPE, "argmax_confidence: too many rows");
  ConfidenceParams p;
  p.out_token = out_token; p.out_conf = out_conf; p.logits = (const char *)logits; p.picks = picks;
  p.V = V; p.row_bytes = row_stride * es;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == ACACHE_BF16) hipLaunchKernelGGL((confidence_kernel<ACACHE_BF16>), dim3((unsigned)R), dim3(kConfThreads), 0, s, p);
  else if (dtype == ACACHE_F16) hipLaunchKernelGGL((confidence_kernel<ACACHE_F16>), dim3((unsigned)R), dim3(kConfThreads), 0, s, p);
  else hipLaunchKernelGGL((confidence_kernel<ACACHE_F32>), dim3((unsigned)R), dim3(kConfThreads), 0, s, p);
  return launch_status("confidence_kernel");
}
