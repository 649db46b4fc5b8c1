// Declarations shared by the attention kernels (gfx950): parameters, relocation modes, the query-tile
// lookups, the global -> LDS copy and the two online-softmax steps.  Everything that must round identically
// in every attention kernel lives here.
#pragma once
#include "common.h"
#include "mma.h"

namespace acache {

enum { MODE_PLAIN = 0, MODE_KEY_SIDE = 1, MODE_QUERY_SIDE = 2 };

// Source of absent rows for the global->LDS copies: a key past the end of its
// range, or one whose slot lies outside the cache, is fetched from here, so the
// LDS tiles are written by the copy engine only (no competing ds_write).
static __device__ __attribute__((aligned(256))) const uint32_t kZeroRow[64] = {0};

struct AttnParams {
  char *out;
  const char *q;
  const char *k_cache;
  const char *v_cache;
  const int32_t *cu_q;
  const int32_t *cu_k;
  const int32_t *slot_map;
  const int32_t *shared_kv_lens;
  const int32_t *affix_shifts;
  const float *cos_tab;
  const float *sin_tab;
  const int32_t *plan;  // optional dispatch plan: (request, tile | head << 20) per block, or NULL
  float scale_log2e;
  int32_t shared_prefix_len;
  int32_t rope_rows;
  int32_t B;
  int32_t H;
  int32_t H_kv;
  int32_t num_tiles;  // upper bound on the number of BM-row query tiles
  int32_t head_dim;   // real head_dim (read by the padded any-head_dim variant only)
  int64_t num_slots;
  int64_t q_token_bytes, q_head_bytes;
  int64_t o_token_bytes, o_head_bytes;
  int64_t kv_slot_bytes, kv_head_bytes;
};

// Which (request, query tile) does global tile index `tile` address?  Lane i loads
// cu_q[i], cu_q[i+1] for 64 requests at a time, an inclusive wave prefix sum of the
// per-request tile counts locates the request with one ballot: one memory round
// trip instead of a dependent scalar load per request.  Returns false when `tile`
// lies beyond the last live tile.  All lanes return the same values.
__device__ __forceinline__ bool locate_query_tile(const int32_t *cu_q, int B, int BM, int tile, int &b_out,
                                                  int &q_begin, int &q_len, int &tile_in_request) {
  const int lane = threadIdx.x & 63;
  int base_tiles = 0;
  for (int b0 = 0; b0 < B; b0 += 64) {
    const int b = b0 + lane;
    const int lo = b < B ? cu_q[b] : 0;
    const int hi = b < B ? cu_q[b + 1] : 0;
    const int len = hi - lo;
    const int tiles = b < B && len > 0 ? (len + BM - 1) / BM : 0;
    int incl = tiles;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const int up = __shfl_up(incl, d);
      if (lane >= d) incl += up;
    }
    const uint64_t hit = __builtin_amdgcn_ballot_w64(base_tiles + incl > tile);
    if (hit != 0) {
      const int src = __builtin_ctzll(hit);
      b_out = b0 + src;
      q_begin = __shfl(lo, src);
      q_len = __shfl(len, src);
      tile_in_request = tile - base_tiles - (__shfl(incl, src) - __shfl(tiles, src));
      return true;
    }
    base_tiles += __shfl(incl, 63);
  }
  return false;
}

// Same lookup, but over the requests sorted by descending key count (ties: lower index first), for
// batches of up to 64 requests.  A block's run time is proportional to its request's key count
// and the hardware hands out blocks in index order, so this is longest-processing-time-first
// list scheduling: the short blocks fill the gaps at the end instead of the long ones sticking out.
__device__ __forceinline__ bool locate_query_tile_lpt(const int32_t *cu_q, const int32_t *cu_k, int B, int BM,
                                                      int rank, int &b_out, int &q_begin, int &q_len,
                                                      int &tile_in_request, int &kv_begin, int &kv_len) {
  const int lane = threadIdx.x & 63;
  // four unconditional loads at a clamped index: one memory round trip (loads under a lane mask end up in
  // separate blocks, each with its own wait)
  const int l = lane < B ? lane : B - 1;
  const int q0 = cu_q[l], q1 = cu_q[l + 1], k0 = cu_k[l], k1 = cu_k[l + 1];
  const int lo = q0;
  const int len = lane < B ? q1 - q0 : 0;
  const int kv = lane < B ? k1 - k0 : 0;
  const int tiles = len > 0 ? (len + BM - 1) / BM : 0;
  int before = 0;  // query tiles of the requests sorted in front of this lane's request
  for (int j = 0; j < B; ++j) {
    const int kv_j = __builtin_amdgcn_readlane(kv, j);
    const int tiles_j = __builtin_amdgcn_readlane(tiles, j);
    if (kv_j > kv || (kv_j == kv && j < lane)) before += tiles_j;
  }
  const uint64_t hit = __builtin_amdgcn_ballot_w64(lane < B && rank >= before && rank < before + tiles);
  if (hit == 0) return false;
  const int src = __builtin_ctzll(hit);
  b_out = src;
  q_begin = __builtin_amdgcn_readlane(lo, src);
  q_len = __builtin_amdgcn_readlane(len, src);
  tile_in_request = rank - __builtin_amdgcn_readlane(before, src);
  kv_begin = __builtin_amdgcn_readlane(k0, src);
  kv_len = __builtin_amdgcn_readlane(kv, src);
  return true;
}

// Block -> (query tile rank, KV head, head inside its group) for the kernels that stream K/V per (tile, head).
// Consecutive block indices go to different XCDs (index mod 8), each with its own L2, so every XCD is given a
// contiguous range of KV heads: all query tiles that read a head's K/V find it in the same L2.
//   H_kv a multiple of 8: an XCD owns H_kv / 8 KV heads, walks the query tiles in its outer loop (in the order
//     the caller's tile lookup defines, longest request first for up to 64 requests) and its heads in the inner one;
//   H_kv = 1, 2 or 4: 8 / H_kv XCDs share a KV head and deal its query tiles out round-robin in that same
//     order, so each of them gets the same mix of long and short tiles;
//   otherwise heads are outermost over one linear index.
// The grid must hold attn_grid_blocks(p) blocks.  Returns false for a block without work.
__device__ __forceinline__ bool block_to_tile_head(const AttnParams &p, int &tile, int &kvh, int &hg) {
  const int per_xcd = gridDim.x >> 3;
  const int xcd = blockIdx.x & 7, idx = blockIdx.x >> 3;
  const int group = p.H / p.H_kv;
  if (p.H_kv % 8 == 0) {
    const int heads_per_xcd = (p.H_kv >> 3) * group;
    tile = idx / heads_per_xcd;
    if (tile >= p.num_tiles) return false;
    const int r = idx - tile * heads_per_xcd;
    kvh = xcd * (p.H_kv >> 3) + r / group;
    hg = r % group;
  } else if (8 % p.H_kv == 0) {
    const int xcds_per_head = 8 / p.H_kv;
    kvh = xcd / xcds_per_head;
    tile = (idx / group) * xcds_per_head + xcd % xcds_per_head;
    if (tile >= p.num_tiles) return false;
    hg = idx % group;
  } else {
    const int w = xcd * per_xcd + idx;
    if (w >= p.num_tiles * p.H) return false;
    hg = w % group;
    tile = (w / group) % p.num_tiles;
    kvh = w / (group * p.num_tiles);
  }
  return true;
}

inline int64_t attn_grid_blocks(const AttnParams &p) {
  if (p.H_kv < 8 && 8 % p.H_kv == 0) {
    const int xcds_per_head = 8 / p.H_kv;
    return 8 * (((int64_t)p.num_tiles + xcds_per_head - 1) / xcds_per_head) * (p.H / p.H_kv);
  }
  return ((int64_t)p.num_tiles * p.H + 7) / 8 * 8;  // the XCD remap needs a multiple of 8
}

// Key range of tile t: the shared range [0, shared_len) comes first in tiles of BN
// (query-side mode only, otherwise shared_len = 0), then [shared_len, kv_len).
struct TileRange {
  int n0, n_end;
};
__device__ __forceinline__ TileRange tile_range_of(int t, int tiles_a, int shared_len, int kv_len, int BN) {
  TileRange r;
  if (t < tiles_a) { r.n0 = t * BN; r.n_end = shared_len; }
  else { r.n0 = shared_len + (t - tiles_a) * BN; r.n_end = kv_len; }
  return r;
}

// Copy 16 bytes per lane from global memory straight into LDS (no register round trip): lane l's
// bytes land at lds_dst + 16*l, lds_dst being wave-uniform.  The copy is counted by vmcnt; the
// caller waits (s_waitcnt vmcnt(0)) and synchronises before anybody reads the bytes.
//
// Issued from inline assembly rather than __builtin_amdgcn_global_load_lds on purpose: while a
// copy the compiler knows about is in flight it treats it as a flat access that may touch both
// memories and turns every later wait for an ordinary LDS read into lgkmcnt(0)/vmcnt(0), which
// serialises the fragment reads of the matrix loops behind one another.  The leading s_nop covers
// the wait state the hardware wants between the write of M0 and its use by the copy.
__device__ __forceinline__ void lds_dma16(const char *src, char *lds_dst) {
  const uint32_t base = __builtin_amdgcn_readfirstlane(
      (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char *)lds_dst);
  asm volatile("s_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(src), "{m0}"(base) : "memory");
}

// The same copy with the destination given as a byte offset inside LDS.  Callers compute it from scalar values
// (the ring buffer's offset, a constant once the buffer pointer is cast BEFORE any lane-derived term is added,
// plus a wave offset taken through readfirstlane once), so the destination costs scalar adds: no 64-bit pointer
// per copy in vector registers, no null check of a generic pointer, no readfirstlane pair per copy.
__device__ __forceinline__ uint32_t lds_offset_of(const char *lds_ptr) {
  return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const char *)lds_ptr;
}
__device__ __forceinline__ void lds_dma16_at(const char *src, uint32_t lds_offset) {
  asm volatile("s_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(src), "{m0}"(lds_offset) : "memory");
}

// A pointer every lane holds the same value of, moved to scalar registers.
__device__ __forceinline__ const char *uniform_ptr(const char *p) {
  const uint64_t v = reinterpret_cast<uint64_t>(p);
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v);
  const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
  return reinterpret_cast<const char *>(((uint64_t)hi << 32) | lo);
}
// The copy with the source given as a wave-uniform base plus a 32-bit byte offset per lane.
__device__ __forceinline__ void lds_dma16_off(const char *base, uint32_t offset, uint32_t lds_offset) {
  asm volatile("s_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(offset), "s"(base), "{m0}"(lds_offset) : "memory");
}

// Online-softmax update of one key tile, in two steps shared by both attention kernels so that
// they round identically (key-side relocation must reproduce a materialised copy bit for bit).
//
// Step 1, softmax_reference: mask absent keys, take the tile's row maxima and move the running
// reference m_run when needed.
//   s_acc  raw scores S^T of the tile (lane: key rows 16*nt + 4*lg + i, query column li)
//   m_run  reference point of the running sums in log2 units (score * scale * log2 e).  It only
//          has to stay within 2^8 of the true running maximum: probabilities up to 256 are
//          harmless in fp32/bf16 and the final division by the running sum cancels the reference.
//          The rescale of O (32 multiplies per lane and query tile) therefore runs only when some
//          query's maximum jumped by more than 8 — one wave-uniform test per tile of 16 queries,
//          rarely true after the first key tile.
//   MASKED keys at tile rows >= n_valid are absent (last tile of a range) and get score -inf.
//   NQA    the first NQA of the wave's NQ16 query tiles are live; the others are left alone
template <int NQA, int NQ16, int NT, int DT, bool MASKED>
__device__ __forceinline__ void softmax_reference(f32x4 (&s_acc)[NQ16][NT], float (&m_run)[NQ16],
                                                  f32x4 (&l_acc)[NQ16], f32x4 (&o_acc)[NQ16][DT],
                                                  float c, int n_valid, int lg) {
  static_assert(NQA <= NQ16, "live query tiles");
#pragma unroll
  for (int qt = 0; qt < NQA; ++qt) {
    if (MASKED && n_valid < 16 * NT) {  // wave-uniform: full tiles skip the masking code
      const int limit = n_valid - 4 * lg;  // one lane-dependent value; the row offsets below are immediates
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (16 * nt + i >= limit) s_acc[qt][nt][i] = -INFINITY;
    }
    float mx = -INFINITY;
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
      for (int i = 0; i < 4; ++i) mx = fmaxf(mx, s_acc[qt][nt][i]);
    // decided per tile of 16 queries, so a query row's arithmetic does not depend on which other rows share
    // its wave (workgroups may give a wave one or two such tiles).  Every lane tests the maximum of its own
    // keys: the ballot is true exactly when some query's maximum over the whole tile exceeds the bound, so the
    // cross-lane maximum (two LDS round trips) is only taken when the reference really moves.
    // (a first tile without any present key still moves the reference off -inf, to 0, so that the
    // probabilities below come out as exp2(-inf) = 0 rather than exp2(-inf + inf))
    if (__builtin_amdgcn_ballot_w64(mx * c > m_run[qt] + 8.0f || m_run[qt] == -INFINITY) != 0) {
      mx = fmaxf(mx, __shfl_xor(mx, 16));
      mx = fmaxf(mx, __shfl_xor(mx, 32));
      const float mxc = mx * c;
      const float m_new = fmaxf(m_run[qt], mxc);
      const float m_use = m_new == -INFINITY ? 0.0f : m_new;
      const float alpha = __builtin_amdgcn_exp2f(m_run[qt] - m_use);
      l_acc[qt] *= alpha;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) o_acc[qt][dt] *= alpha;
      m_run[qt] = m_use;
    }
  }
}

// Step 2, softmax_probs_slab: probabilities of the 32-key slab S of the tile, packed as the B
// operand pf[qt][S] of the PV product, and their contribution to the softmax denominator.
// l_acc is accumulated by the matrix core as one more row block of O^T whose V^T rows are all
// ones: every element of l_acc[qt] ends up holding sum_n P[n][query li] of the ROUNDED
// probabilities, with no VALU adds or cross-lane reduction.  Slabs must be taken in order.
template <class M, int S, int NQA, int NQ16, int NT, int NS>
__device__ __forceinline__ void softmax_probs_slab(const f32x4 (&s_acc)[NQ16][NT], const float (&m_run)[NQ16],
                                                   f32x4 (&l_acc)[NQ16], vec16 (&pf)[NQ16][NS],
                                                   const vec16 &ones, float c) {
#pragma unroll
  for (int qt = 0; qt < NQA; ++qt) {
    const float mc = m_run[qt];
    float e[8];
#pragma unroll
    // one fused multiply-add per score (contraction is switched off for this library, so it is asked for by name)
    for (int j = 0; j < 8; ++j) e[j] = __builtin_amdgcn_exp2f(__builtin_fmaf(s_acc[qt][2 * S + (j >> 2)][j & 3], c, -mc));
    pf[qt][S].w[0] = M::pack2(e[0], e[1]);
    pf[qt][S].w[1] = M::pack2(e[2], e[3]);
    pf[qt][S].w[2] = M::pack2(e[4], e[5]);
    pf[qt][S].w[3] = M::pack2(e[6], e[7]);
    l_acc[qt] = M::run(ones, pf[qt][S], l_acc[qt]);
  }
}

}  // namespace acache
