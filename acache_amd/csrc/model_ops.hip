// Two elementwise steps of the decoder block around the attention path (gfx950), used by the package's own
// LLaDA / Dream model mirror: SwiGLU on the merged gate / up projection, and residual add + RMSNorm.
// Both are bound by HBM: every element is read once and written once, 16 bytes per lane.
#include "common.h"

namespace acache {

// out[t, j] = silu(gu[t, j]) * gu[t, m + j]: the gate half and the up half of one projection row.
// silu(x) = x / (1 + exp(-x)) in fp32, rounded to the storage type, then multiplied by the up value in
// fp32 and rounded again: the two roundings of the separate activation and multiply kernels.
template <int DTYPE>
__global__ __launch_bounds__(256) void swiglu_kernel(char *out, const char *gu, int64_t chunks_per_row,
                                                     int64_t total_chunks, int64_t in_row_bytes,
                                                     int64_t out_row_bytes, int64_t half_bytes) {
  using E = Elem<DTYPE>;
  constexpr int VEC = E::kPerVec;
  const int64_t c = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (c >= total_chunks) return;
  const int64_t row = c / chunks_per_row;
  const int64_t col = c - row * chunks_per_row;
  const char *src = gu + row * in_row_bytes + col * 16;
  float g[VEC], u[VEC], y[VEC];
  E::unpack(load16_stream(src), g);
  E::unpack(load16_stream(src + half_bytes), u);
#pragma unroll
  for (int j = 0; j < VEC; ++j) y[j] = g[j] / (1.0f + __expf(-g[j]));
  const vec16 act = E::pack(y);  // first rounding: the activation's own output
  E::unpack(act, y);
#pragma unroll
  for (int j = 0; j < VEC; ++j) y[j] *= u[j];
  store16(out + row * out_row_bytes + col * 16, E::pack(y));
}

// sum[t, :] = x[t, :] + delta[t, :] (rounded to the storage type),
// y[t, :]   = round(sum[t, :] * rsqrt(mean(sum[t, :]^2) + eps)) * w[:]: statistics in fp32, the normalised value
// rounded to the storage type before the weight multiplies it and the product rounded again, which is where the
// reference's layer norm rounds (llada/model/modeling_llada.py:338-350: x.to(og_dtype), then weight * x).
// Without delta the sum is x itself and is not written.  One 256-thread block per row; a thread keeps its
// chunks of the row in registers between the two steps (rows of up to 256 * 16 bytes * kMaxChunks).
constexpr int kMaxChunks = 4;

template <int DTYPE>
__global__ __launch_bounds__(256) void add_rms_norm_kernel(char *sum, const char *x, const char *delta,
                                                           const char *weight, char *y, int chunks_per_row,
                                                           int64_t sum_row_bytes, int64_t x_row_bytes,
                                                           int64_t delta_row_bytes, int64_t y_row_bytes, float eps,
                                                           float inv_d) {
  using E = Elem<DTYPE>;
  constexpr int VEC = E::kPerVec;
  const int tid = threadIdx.x;
  const char *xr = x + (int64_t)blockIdx.x * x_row_bytes;
  char *sr = sum + (int64_t)blockIdx.x * sum_row_bytes;
  const char *dr = delta ? delta + (int64_t)blockIdx.x * delta_row_bytes : nullptr;
  char *yr = y + (int64_t)blockIdx.x * y_row_bytes;
  float v[kMaxChunks][VEC];
  float ss = 0.0f;
#pragma unroll
  for (int i = 0; i < kMaxChunks; ++i) {
    const int c = tid + i * 256;
    if (c < chunks_per_row) {
      E::unpack(load16(xr + c * 16), v[i]);
      if (dr) {
        float d[VEC];
        E::unpack(load16_stream(dr + c * 16), d);
#pragma unroll
        for (int j = 0; j < VEC; ++j) v[i][j] += d[j];
        const vec16 rounded = E::pack(v[i]);  // the residual stream keeps the rounded sum
        store16(sr + c * 16, rounded);
        E::unpack(rounded, v[i]);
      }
#pragma unroll
      for (int j = 0; j < VEC; ++j) ss += v[i][j] * v[i][j];
    }
  }
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) ss += __shfl_xor(ss, d);
  __shared__ float part[4];
  if ((tid & 63) == 0) part[tid >> 6] = ss;
  __syncthreads();
  const float scale = rsqrtf((part[0] + part[1] + part[2] + part[3]) * inv_d + eps);
#pragma unroll
  for (int i = 0; i < kMaxChunks; ++i) {
    const int c = tid + i * 256;
    if (c < chunks_per_row) {
      float w[VEC], o[VEC];
      E::unpack(load16(weight + c * 16), w);
#pragma unroll
      for (int j = 0; j < VEC; ++j) o[j] = v[i][j] * scale;
      E::unpack(E::pack(o), o);  // the normalised row in the storage type
#pragma unroll
      for (int j = 0; j < VEC; ++j) o[j] *= w[j];
      store16(yr + c * 16, E::pack(o));
    }
  }
}

}  // namespace acache

using namespace acache;

extern "C" int acache_swiglu(void *out, const void *gate_up, int64_t M, int64_t m, int64_t in_row_stride,
                             int64_t out_row_stride, int32_t dtype, void *stream) {
  const int es = dtype_bytes(dtype);
  if (es == 0) return fail(ACACHE_E_DTYPE, "swiglu: unknown dtype %d", dtype);
  if (M < 0 || m <= 0) return fail(ACACHE_E_SHAPE, "swiglu: M %lld, m %lld", (long long)M, (long long)m);
  if (M == 0) return 0;
  if (!out || !gate_up) return fail(ACACHE_E_NULL, "swiglu: NULL pointer");
  if (in_row_stride < 2 * m || out_row_stride < m) return fail(ACACHE_E_SHAPE, "swiglu: row stride smaller than a row");
  if ((m * es) % 16 || (in_row_stride * es) % 16 || (out_row_stride * es) % 16 || !aligned16(out) || !aligned16(gate_up))
    return fail(ACACHE_E_ALIGN, "swiglu: rows, halves and pointers must be 16-byte aligned");
  const int64_t cpr = m * es / 16, total = cpr * M;
  const int64_t blocks = (total + 255) / 256;
  if (blocks > 0x7fffffffLL) return fail(ACACHE_E_SHAPE, "swiglu: too many elements");
  hipStream_t s = (hipStream_t)stream;
#define ACACHE_CASE(DT)                                                                                          \
  if (dtype == DT) {                                                                                             \
    hipLaunchKernelGGL((swiglu_kernel<DT>), dim3((unsigned)blocks), dim3(256), 0, s, (char *)out,                \
                       (const char *)gate_up, cpr, total, in_row_stride * es, out_row_stride * es, m * es);      \
    return launch_status("swiglu_kernel");                                                                       \
  }
  ACACHE_CASE(ACACHE_BF16)
  ACACHE_CASE(ACACHE_F16)
  ACACHE_CASE(ACACHE_F32)
#undef ACACHE_CASE
  return fail(ACACHE_E_DTYPE, "swiglu: unknown dtype %d", dtype);
}

extern "C" int acache_add_rms_norm(void *sum, const void *x, const void *delta, const void *weight, void *y,
                                   int64_t M, int64_t d, int64_t sum_row_stride, int64_t x_row_stride,
                                   int64_t delta_row_stride, int64_t y_row_stride, float eps, int32_t dtype,
                                   void *stream) {
  const int es = dtype_bytes(dtype);
  if (es == 0) return fail(ACACHE_E_DTYPE, "add_rms_norm: unknown dtype %d", dtype);
  if (M < 0 || d <= 0) return fail(ACACHE_E_SHAPE, "add_rms_norm: M %lld, d %lld", (long long)M, (long long)d);
  if (M == 0) return 0;
  if (!x || !weight || !y || (delta && !sum)) return fail(ACACHE_E_NULL, "add_rms_norm: NULL pointer");
  if ((d * es) % 16 || d * es / 16 > 256 * kMaxChunks)
    return fail(ACACHE_E_SHAPE, "add_rms_norm: row of %lld elements not supported (16-byte multiple, at most %d bytes)",
                (long long)d, 256 * kMaxChunks * 16);
  if (x_row_stride < d || y_row_stride < d || (delta && (delta_row_stride < d || sum_row_stride < d)))
    return fail(ACACHE_E_SHAPE, "add_rms_norm: row stride smaller than a row");
  if (!aligned16(x) || !aligned16(weight) || !aligned16(y) || (x_row_stride * es) % 16 || (y_row_stride * es) % 16 ||
      (delta && (!aligned16(delta) || !aligned16(sum) || (delta_row_stride * es) % 16 || (sum_row_stride * es) % 16)))
    return fail(ACACHE_E_ALIGN, "add_rms_norm: pointers and row strides must be 16-byte aligned");
  if (!(eps >= 0.0f)) return fail(ACACHE_E_RANGE, "add_rms_norm: eps must be non-negative");
  if (M > 0x7fffffffLL) return fail(ACACHE_E_SHAPE, "add_rms_norm: too many rows");
  hipStream_t s = (hipStream_t)stream;
  const int cpr = (int)(d * es / 16);
#define ACACHE_CASE(DT)                                                                                          \
  if (dtype == DT) {                                                                                             \
    hipLaunchKernelGGL((add_rms_norm_kernel<DT>), dim3((unsigned)M), dim3(256), 0, s, (char *)sum,               \
                       (const char *)x, (const char *)delta, (const char *)weight, (char *)y, cpr,               \
                       sum_row_stride * es, x_row_stride * es, delta_row_stride * es, y_row_stride * es, eps,    \
                       1.0f / (float)d);                                                                         \
    return launch_status("add_rms_norm_kernel");                                                                 \
  }
  ACACHE_CASE(ACACHE_BF16)
  ACACHE_CASE(ACACHE_F16)
  ACACHE_CASE(ACACHE_F32)
#undef ACACHE_CASE
  return fail(ACACHE_E_DTYPE, "add_rms_norm: unknown dtype %d", dtype);
}
