// Scatter of recomputed K/V rows into the paged cache, and block-table -> slot
// expansion (gfx950).
//
// A token record is H_kv*D contiguous elements; it is moved as 16-byte chunks,
// consecutive lanes on consecutive chunks, so a 1 KiB Dream record (H_kv = 4,
// D = 128, bf16) is one wave64 store and an 8 KiB LLaDA record is two blocks'
// worth of fully coalesced stores.  All layers go in one launch (grid.y).
// HBM traffic per row and layer: 2 (K,V) * 2 (read+write) * H_kv * D * bytes.
#include "common.h"

namespace acache {

struct ScatterParams {
  char *k_cache;
  char *v_cache;
  const char *key;
  const char *value;
  const int32_t *slot_map;
  int64_t N;
  int64_t num_slots;
  int64_t key_token_bytes;
  int64_t value_token_bytes;
  int64_t src_layer_bytes;
  int64_t cache_layer_bytes;
  int32_t chunks_per_token;  // H_kv * D * bytes / 16
  int32_t L;
};

// STREAM: non-temporal stores.  A launch that writes more than the L2 holds gains 13 % from them (68 -> 59 us
// for 166 MB of rows into shuffled blocks); a small one keeps ordinary stores, so that the attention call
// behind it finds the fresh rows in L2.
template <int LPB, bool STREAM>
__global__ __launch_bounds__(256) void scatter_kernel(ScatterParams p) {
  const int64_t gid = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int64_t token = gid / p.chunks_per_token;
  if (token >= p.N) return;
  const int chunk = (int)(gid - token * p.chunks_per_token);
  const int64_t slot = p.slot_map[token];
  if (slot < 0 || slot >= p.num_slots) return;  // -1 = "do not store"
  const int l0 = blockIdx.y * LPB;
  const int64_t dst = slot * p.chunks_per_token * 16 + (int64_t)chunk * 16;
  const int64_t ksrc = token * p.key_token_bytes + (int64_t)chunk * 16;
  const int64_t vsrc = token * p.value_token_bytes + (int64_t)chunk * 16;
  vec16 k[LPB], v[LPB];
#pragma unroll
  for (int i = 0; i < LPB; ++i) {
    if (l0 + i < p.L) {
      k[i] = load16_stream(p.key + (int64_t)(l0 + i) * p.src_layer_bytes + ksrc);
      v[i] = load16_stream(p.value + (int64_t)(l0 + i) * p.src_layer_bytes + vsrc);
    }
  }
#pragma unroll
  for (int i = 0; i < LPB; ++i) {
    if (l0 + i < p.L) {
      char *const kd = p.k_cache + (int64_t)(l0 + i) * p.cache_layer_bytes + dst;
      char *const vd = p.v_cache + (int64_t)(l0 + i) * p.cache_layer_bytes + dst;
      if (STREAM) { store16_stream(kd, k[i]); store16_stream(vd, v[i]); }
      else { store16(kd, k[i]); store16(vd, v[i]); }
    }
  }
}

__global__ __launch_bounds__(256) void block_table_slots_kernel(
    int32_t *out, const int32_t *tables, const int32_t *cu_k, int B, int max_blocks,
    int block_size) {
  const int b = blockIdx.y;
  const int start = cu_k[b];
  const int len = cu_k[b + 1] - start;
  for (int n = blockIdx.x * 256 + threadIdx.x; n < len; n += gridDim.x * 256) {
    const int blk = n / block_size;
    // a request longer than its table is a caller bug; map it to slot -1
    // (readers turn out-of-range slots into zero rows) instead of reading past it
    const int id = blk < max_blocks ? tables[(int64_t)b * max_blocks + blk] : -1;
    out[start + n] = id < 0 ? -1 : id * block_size + (n - blk * block_size);
  }
}

// Slot layout of a batch of requests with a reused affix, one thread per token: where attention reads each
// position from, and the (position, slot) list of the tokens that are recomputed (anchors + everything outside
// the affix), in position order.  A request's private slots are enumerated block by block from its block table:
// the first K go to its anchors in ascending position order, the rest to the non-affix positions in order.
struct SlotLayoutParams {
  int32_t *read_slots;
  int32_t *recompute_pos;
  int32_t *recompute_slots;
  const int32_t *cu_len;
  const int32_t *cu_rec;
  const int32_t *affix_start;
  const int32_t *affix_end;
  const int32_t *cu_anchor;
  const int32_t *anchors;
  const int32_t *tables;
  int32_t max_blocks;
  int32_t block_size;
  int32_t shared_slot_offset;
};

__global__ __launch_bounds__(256) void slot_layout_kernel(SlotLayoutParams p) {
  const int b = blockIdx.y;
  const int t0 = p.cu_len[b];
  const int len = p.cu_len[b + 1] - t0;
  const int a_lo = p.affix_start[b], a_hi = p.affix_end[b];
  const int k0 = p.cu_anchor[b];
  const int K = p.cu_anchor[b + 1] - k0;
  const int r0 = p.cu_rec[b];
  const int rec_len = p.cu_rec[b + 1] - r0;  // K + len - (a_hi - a_lo) when the inputs are consistent
  const int32_t *anc = p.anchors + k0;
  for (int pos = blockIdx.x * 256 + threadIdx.x; pos < len; pos += gridDim.x * 256) {
    int priv = -1, rank = -1;
    if (pos >= a_lo && pos < a_hi) {
      int lo = 0, hi = K;  // first anchor >= pos
      while (lo < hi) {
        const int mid = (lo + hi) >> 1;
        if (anc[mid] < pos) lo = mid + 1; else hi = mid;
      }
      if (lo < K && anc[lo] == pos) { priv = lo; rank = a_lo + lo; }
    } else if (pos < a_lo) {
      priv = K + pos; rank = pos;
    } else {
      priv = K + pos - (a_hi - a_lo); rank = a_lo + K + (pos - a_hi);
    }
    int slot;
    if (priv < 0) {
      slot = p.shared_slot_offset + (pos - a_lo);  // frozen affix token: the shared copy
    } else {
      const int blk = priv / p.block_size;
      const int id = blk < p.max_blocks ? p.tables[(int64_t)b * p.max_blocks + blk] : -1;
      slot = id < 0 ? -1 : id * p.block_size + (priv - blk * p.block_size);
      if (rank < rec_len) {  // never write past this request's share, whatever the anchor list holds
        p.recompute_pos[r0 + rank] = pos;
        p.recompute_slots[r0 + rank] = slot;
      }
    }
    p.read_slots[t0 + pos] = slot;
  }
}

}  // namespace acache

using namespace acache;

extern "C" int acache_kv_scatter(
    void *k_cache, void *v_cache, const void *key, const void *value, const int32_t *slot_map,
    int64_t N, int32_t L, int32_t H_kv, int32_t D, int32_t dtype, int64_t num_slots,
    int64_t key_token_stride, int64_t value_token_stride, int64_t src_layer_stride,
    int64_t cache_layer_stride, void *stream) {
  const int es = dtype_bytes(dtype);
  if (es == 0) return fail(ACACHE_E_DTYPE, "kv_scatter: unknown dtype %d", dtype);
  if (N < 0 || L < 0 || H_kv <= 0 || D <= 0 || num_slots < 0)
    return fail(ACACHE_E_SHAPE, "kv_scatter: negative size");
  if (N == 0 || L == 0) return 0;
  if (!k_cache || !v_cache || !key || !value || !slot_map)
    return fail(ACACHE_E_NULL, "kv_scatter: NULL pointer");
  const int64_t tok = (int64_t)H_kv * D;
  if ((tok * es) % 16) return fail(ACACHE_E_SHAPE, "kv_scatter: H_kv*D*bytes must be a multiple of 16");
  if (key_token_stride < tok || value_token_stride < tok)
    return fail(ACACHE_E_SHAPE, "kv_scatter: token stride smaller than H_kv*D");
  if (!aligned16(k_cache) || !aligned16(v_cache) || !aligned16(key) || !aligned16(value) ||
      (key_token_stride * es) % 16 || (value_token_stride * es) % 16 ||
      (L > 1 && ((src_layer_stride * es) % 16 || (cache_layer_stride * es) % 16)))
    return fail(ACACHE_E_ALIGN, "kv_scatter: pointers and strides must be 16-byte aligned");
  if (L > 1 && cache_layer_stride < num_slots * tok)
    return fail(ACACHE_E_SHAPE, "kv_scatter: cache layer stride smaller than one layer");
  ScatterParams p;
  p.k_cache = (char *)k_cache; p.v_cache = (char *)v_cache;
  p.key = (const char *)key; p.value = (const char *)value; p.slot_map = slot_map;
  p.N = N; p.num_slots = num_slots;
  p.key_token_bytes = key_token_stride * es; p.value_token_bytes = value_token_stride * es;
  p.src_layer_bytes = src_layer_stride * es; p.cache_layer_bytes = cache_layer_stride * es;
  p.chunks_per_token = (int32_t)(tok * es / 16); p.L = L;
  const int64_t gx = (N * p.chunks_per_token + 255) / 256;
  constexpr int LPB = 2;
  if (gx > 0x7fffffffLL || (L + LPB - 1) / LPB > 65535) return fail(ACACHE_E_SHAPE, "kv_scatter: too many rows or layers");
  dim3 grid((unsigned)gx, (unsigned)((L + LPB - 1) / LPB));
  // rows written by one launch, K and V: beyond 32 MiB (eight times the 4 MiB L2 of an XCD) they stream
  const bool stream_stores = N * tok * es * 2 * L > (32LL << 20);
  if (stream_stores) hipLaunchKernelGGL((scatter_kernel<LPB, true>), grid, dim3(256), 0, (hipStream_t)stream, p);
  else hipLaunchKernelGGL((scatter_kernel<LPB, false>), grid, dim3(256), 0, (hipStream_t)stream, p);
  return launch_status("scatter_kernel");
}

extern "C" int acache_block_table_slots(
    int32_t *out_slots, const int32_t *block_tables, const int32_t *cu_k, int32_t B,
    int32_t max_blocks, int32_t block_size, int64_t total_k, void *stream) {
  if (B < 0 || max_blocks < 0 || block_size <= 0 || total_k < 0)
    return fail(ACACHE_E_SHAPE, "block_table_slots: bad size");
  if (B == 0 || total_k == 0) return 0;
  if (!out_slots || !block_tables || !cu_k) return fail(ACACHE_E_NULL, "block_table_slots: NULL pointer");
  if (B > 65535) return fail(ACACHE_E_SHAPE, "block_table_slots: batch %d > 65535", B);
  int64_t gx = (total_k / B + 255) / 256 + 1;
  if (gx > 1024) gx = 1024;
  hipLaunchKernelGGL(block_table_slots_kernel, dim3((unsigned)gx, (unsigned)B), dim3(256), 0,
                     (hipStream_t)stream, out_slots, block_tables, cu_k, B, max_blocks, block_size);
  return launch_status("block_table_slots_kernel");
}

extern "C" int acache_build_slot_layout(
    int32_t *read_slots, int32_t *recompute_pos, int32_t *recompute_slots, const int32_t *cu_len,
    const int32_t *cu_rec, const int32_t *affix_start, const int32_t *affix_end, const int32_t *cu_anchor,
    const int32_t *anchors, const int32_t *block_tables, int32_t B, int32_t max_blocks, int32_t block_size,
    int32_t shared_slot_offset, int64_t total_tokens, void *stream) {
  if (B < 0 || max_blocks < 0 || block_size <= 0 || total_tokens < 0 || shared_slot_offset < 0)
    return fail(ACACHE_E_SHAPE, "build_slot_layout: bad size");
  if (B == 0 || total_tokens == 0) return 0;
  if (!read_slots || !recompute_pos || !recompute_slots || !cu_len || !cu_rec || !affix_start || !affix_end ||
      !cu_anchor || !block_tables)
    return fail(ACACHE_E_NULL, "build_slot_layout: NULL pointer");
  if (B > 65535) return fail(ACACHE_E_SHAPE, "build_slot_layout: batch %d > 65535", B);
  int64_t gx = (total_tokens / B + 255) / 256 + 1;
  if (gx > 1024) gx = 1024;
  SlotLayoutParams p;
  p.read_slots = read_slots; p.recompute_pos = recompute_pos; p.recompute_slots = recompute_slots;
  p.cu_len = cu_len; p.cu_rec = cu_rec; p.affix_start = affix_start; p.affix_end = affix_end;
  p.cu_anchor = cu_anchor; p.anchors = anchors; p.tables = block_tables;
  p.max_blocks = max_blocks; p.block_size = block_size; p.shared_slot_offset = shared_slot_offset;
  hipLaunchKernelGGL(slot_layout_kernel, dim3((unsigned)gx, (unsigned)B), dim3(256), 0, (hipStream_t)stream, p);
  return launch_status("slot_layout_kernel");
}
