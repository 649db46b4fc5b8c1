// Affix importance for anchor selection (gfx950): for every request, the attention that its [MASK]
// queries pay to each cached affix key, soft-maxed over the affix keys only and summed over the mask
// queries and heads of one layer.
//
//   w[r, h, a]       = softmax_a( q[r, h] . rot(K[a, kv(h)], shift_b) * scale )     a in [0, A)
//   importance[b, a] += sum_{r in mask rows of b} sum_h w[r, h, a]
//
// Relocation is applied on the query side: q . rot(k, +s) = rot(q, -s) . k.  A first launch writes each request's
// [MASK] queries, packed in mask-row order and (with relocation) rotated by minus the request's shift, into the
// workspace (a few hundred rows per request); every launch after it reads that copy without an index in between
// and the cached affix keys as they lie in the cache: one copy of the keys, shared by all requests and resident
// in L2, instead of one re-rotated copy per request.  Three more launches, no atomics, so the result does not
// depend on scheduling:
//   1. statistics pass: the mask rows of a wave stay in registers, the affix keys stream by, and the wave
//      leaves log2 of each row's sum of 2^(score * c) in the workspace;
//   2. column pass: the affix keys of a wave stay in registers, the request's mask rows stream by, the scores
//      are recomputed, normalised with the stored row statistic (one subtraction in the exponent) and summed
//      per key; each wave is the only writer of its entries of the per-head partial sums in the workspace;
//   3. importance_reduce_kernel adds the per-head partial sums, in head order, to importance[b, :].
// Scores come from the matrix core (S^T = K Q^T, keys as rows, one query column per lane).  Both passes exist
// twice: for head dims of 64, 128 and 256 the streamed operand is staged through LDS by the copy engine and
// shared by the four waves of a workgroup (importance_*_lds_kernel, further down); every other head dim loads
// its fragments straight from global memory in operand layout, 16 bytes per lane, without LDS or barriers
// (importance_stats_kernel, importance_colsum_kernel).
#include <mutex>
#include <type_traits>

#include "common.h"
#include "mma.h"
#include "attn_common.h"

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
  float *stats;            // per (mask row, head): log2 of the row's sum of 2^(score * c)
  float *partial;
  char *q_rot;            // [total_mask_rows, H, D] mask queries packed in mask-row order, counter-rotated
  int64_t total_q;        // rows of q; a mask row outside [0, total_q) is an absent query
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
  int32_t D;  // head_dim
  int32_t total_mask_rows;  // entries of mask_rows, rows of the packed query copy and of stats
  int32_t max_mask_rows;    // the launch grids cover this many mask rows per request
};

// First mask row and number of mask rows of request b, held to what the workspace and the launch grids were
// sized for: the prefix sums live in device memory, where the host cannot check them, and a request that
// claims more rows than the caller declared is cut there instead of being read past the buffers.
__device__ __forceinline__ void request_rows(const ImportanceParams &p, int b, int &m0, int &n_rows) {
  m0 = p.cu_mask[b];
  m0 = m0 < 0 ? 0 : (m0 > p.total_mask_rows ? p.total_mask_rows : m0);
  int n = p.cu_mask[b + 1] - m0;
  const int room = p.total_mask_rows - m0;
  n = n > room ? room : n;
  n = n > p.max_mask_rows ? p.max_mask_rows : n;
  n_rows = n < 0 ? 0 : n;
}

// Operand fragments of 16 rows x D, KS = ceil(D / 32) slabs of 32 elements: lane (li, lg) takes elements
// 32*ks + 8*lg .. + 8 of row `row_ptr` (always a readable row: callers clamp indices instead of branching, so
// the loads of a tile issue back to back); chunks at or past D (a multiple of 16) read as zeros.
template <int D>
__device__ __forceinline__ void load_rows(vec16 (&f)[(D + 31) / 32], const char *row_ptr, int lg) {
  constexpr int KS = (D + 31) / 32;
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    if (32 * ks + 32 <= D) {
      f[ks] = load16(row_ptr + (32 * ks + 8 * lg) * 2);
    } else {  // the half-filled last slab of D = 16 (mod 32): lane groups 2 and 3 hold zeros
      const vec16 v = load16(row_ptr + (32 * ks + 8 * (lg & 1)) * 2);
      f[ks] = lg < 2 ? v : vec16{{0, 0, 0, 0}};
    }
  }
}

// Counter-rotate the [MASK] queries once per call: q_rot[m0_b + r, h, :] = rot(q[mask_rows[m0_b + r], h, :], -shift_b).
// One row of D elements per D/16 lanes, the rotate-half partner in the same lane; fp32 products and sum rounded
// separately, one rounding to the query type (the query-side arithmetic of the attention kernel).  A mask row
// outside q is written as zeros (and counted as absent by the statistics kernel).
template <int DTYPE>
__global__ __launch_bounds__(256) void importance_rotate_kernel(ImportanceParams p) {
  const int D = p.D;
  const int half_bytes = D;  // D / 2 elements of 2 bytes
  const int lpr = half_bytes / 16;
  const int b = blockIdx.y;
  int m0, n_rows;
  request_rows(p, b, m0, n_rows);
  const int64_t g = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int64_t row = g / lpr;
  const int lane = (int)(g - row * lpr);
  if (row >= (int64_t)n_rows * p.H) return;
  const int r = (int)(row / p.H);
  const int h = (int)(row - (int64_t)r * p.H);
  char *dst = p.q_rot + (((int64_t)(m0 + r) * p.H + h) * D) * 2 + lane * 16;
  const int64_t src_row = p.mask_rows[m0 + r];
  vec16 lo = {{0, 0, 0, 0}}, hi = {{0, 0, 0, 0}};
  if (src_row >= 0 && src_row < p.total_q) {
    const char *src = p.q + src_row * p.q_token_bytes + (int64_t)h * p.q_head_bytes + lane * 16;
    lo = load16(src);
    hi = load16(src + half_bytes);
    int shift = p.shifts ? p.shifts[b] : 0;
    if (shift < 0 || shift >= p.rope_rows) shift = 0;
    if (shift != 0)
      rotate_pair_half<DTYPE>(lo, hi, p.cos_tab + (int64_t)shift * D, p.sin_tab + (int64_t)shift * D, lane * 8, D / 2, -1.0f);
  }
  store16(dst, lo);
  store16(dst + half_bytes, hi);
}

// Row r of request b (first mask row m0), head h, in the packed copy the first launch wrote.  Always a readable
// address: r is clamped to the request's rows (callers discard what a clamped row contributes).  The copy is
// smaller than 4 GiB (checked at launch), so the offset is 32-bit arithmetic.
__device__ __forceinline__ const char *mask_query_row(const ImportanceParams &p, int m0, int n_rows, int r, int h) {
  r = r < n_rows ? r : n_rows - 1;
  return p.q_rot + ((uint32_t)(m0 + r) * (uint32_t)p.H + (uint32_t)h) * (uint32_t)(p.D * 2);
}

// Sum over the 16 lanes of a row (lanes sharing lane >> 4), left in every lane of the row: four rotate-and-add
// steps in the vector ALU's lane-permute path (no trip through LDS).
__device__ __forceinline__ float row_sum16(float v) {
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x128, 0xf, 0xf, false));
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x124, 0xf, 0xf, false));
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x122, 0xf, 0xf, false));
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x121, 0xf, 0xf, false));
  return v;
}

constexpr int kKeysPerStep = 64;  // keys a colsum wave owns (four independent 16-key tiles in flight)
constexpr int kStatKeys = 32;     // keys a stats wave scores per loop step (two 16-key tiles x two row tiles in flight)

constexpr int kRowTilesPerWave = 4;  // 16-row tiles of mask queries a stats wave owns (keys are loaded once for all)

// One wave per (request, head, 64 mask rows): the rows stay in registers, the affix keys stream by, and the wave
// leaves log2(sum_a 2^(s[r, a] * c)) per row (running maximum + log2 of the running sum) in the workspace.
template <int DTYPE, int D>
__global__ __launch_bounds__(256) void importance_stats_kernel(ImportanceParams p) {
  constexpr int NQ = kRowTilesPerWave;
  constexpr int KS = (D + 31) / 32;
  using M = Mma<DTYPE>;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int li = lane & 15, lg = lane >> 4;
  const int groups = (p.max_row_tiles + NQ - 1) / NQ;
  const int b = blockIdx.x / groups, rg = blockIdx.x % groups;
  const int h = blockIdx.y * 4 + wave;
  int m0, n_rows;
  request_rows(p, b, m0, n_rows);
  const int row0 = rg * NQ * 16;
  if (h >= p.H || row0 >= n_rows) return;  // no barrier in this kernel: waves may leave early
  const int kvh = h / (p.H / p.H_kv);

  vec16 qf[NQ][KS];
#pragma unroll
  for (int qt = 0; qt < NQ; ++qt) load_rows<D>(qf[qt], mask_query_row(p, m0, n_rows, row0 + 16 * qt + li, h), lg);
  const char *k_base = p.k_cache + p.affix_slot0 * p.kv_slot_bytes + (int64_t)kvh * p.kv_head_bytes;
  const float c = p.scale_log2e;

  float m_run[NQ], l_run[NQ];  // per query column (lane li); l is this lane group's share
#pragma unroll
  for (int qt = 0; qt < NQ; ++qt) { m_run[qt] = -INFINITY; l_run[qt] = 0.0f; }
  constexpr int NT = kStatKeys / 16;
  // keys a0 + 16*nt + li of one step, clamped to the affix (a clamped key is masked out below)
  auto fetch = [&](int a0, vec16 (&kf)[NT][KS]) __attribute__((always_inline)) {
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      const int a = a0 + 16 * nt + li;
      load_rows<D>(kf[nt], k_base + (int64_t)(a < p.A ? a : p.A - 1) * p.kv_slot_bytes, lg);
    }
  };
  // one step on the keys in `kf`, with the next step's keys requested first (always: past the end the clamped
  // addresses are re-read and the result ignored, which keeps the loop free of a branch the loads would wait at)
  auto step = [&](int a0, vec16 (&kf)[NT][KS], vec16 (&kf_next)[NT][KS]) __attribute__((always_inline)) {
    fetch(a0 + kStatKeys, kf_next);
    const bool tail = a0 + kStatKeys > p.A;  // wave-uniform: only the last step holds keys past the affix
#pragma unroll
    for (int qp = 0; qp < NQ; qp += 2) {  // two row tiles at a time: four independent accumulator chains
      f32x4 sc[2][NT];
#pragma unroll
      for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) sc[u][nt] = f32x4{0, 0, 0, 0};
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
          for (int nt = 0; nt < NT; ++nt) sc[u][nt] = M::run(kf[nt][ks], qf[qp + u][ks], sc[u][nt]);
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        const int qt = qp + u;
        if (tail) {
#pragma unroll
          for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int i = 0; i < 4; ++i)
              if (a0 + 16 * nt + 4 * lg + i >= p.A) sc[u][nt][i] = -INFINITY;
        }
        float mx = -INFINITY;
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
          for (int i = 0; i < 4; ++i) mx = fmaxf(mx, sc[u][nt][i]);
        mx = fmaxf(mx, __shfl_xor(mx, 16));
        mx = fmaxf(mx, __shfl_xor(mx, 32));
        const float m_new = fmaxf(m_run[qt], mx * c);  // finite: every step holds at least one existing key
        float add = 0.0f;
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
          for (int i = 0; i < 4; ++i) add += __builtin_amdgcn_exp2f(__builtin_fmaf(sc[u][nt][i], c, -m_new));
        l_run[qt] = l_run[qt] * __builtin_amdgcn_exp2f(m_run[qt] - m_new) + add;
        m_run[qt] = m_new;
      }
    }
  };
  vec16 kf_a[NT][KS], kf_b[NT][KS];
  fetch(0, kf_a);
  for (int a0 = 0; a0 < p.A; a0 += 2 * kStatKeys) {
    step(a0, kf_a, kf_b);
    if (a0 + kStatKeys < p.A) step(a0 + kStatKeys, kf_b, kf_a);
  }
#pragma unroll
  for (int qt = 0; qt < NQ; ++qt) {
    float l = l_run[qt];
    l += __shfl_xor(l, 16);
    l += __shfl_xor(l, 32);
    const int r = row0 + 16 * qt + li;
    if (lg == 0 && r < n_rows) {
      const int64_t src_row = p.mask_rows[m0 + r];
      const bool present = src_row >= 0 && src_row < p.total_q;  // an absent query gets 2^-inf = 0: it adds nothing
      p.stats[(int64_t)(m0 + r) * p.H + h] = present ? m_run[qt] + __builtin_amdgcn_logf(l) : INFINITY;
    }
  }
}

constexpr int kColRowTiles = 2;  // 16-row tiles of mask queries a colsum wave scores per loop step

// One wave per (request, head, 64 affix keys): the keys stay in registers, the request's mask rows stream by
// 32 at a time (the next 32 already on their way).  The wave is the only writer of partial[b, h, a0 .. a0 + 64).
template <int DTYPE, int D>
__global__ __launch_bounds__(256) void importance_colsum_kernel(ImportanceParams p) {
  constexpr int KS = (D + 31) / 32;
  constexpr int NR = kColRowTiles;
  using M = Mma<DTYPE>;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int li = lane & 15, lg = lane >> 4;
  const int b = blockIdx.z;
  const int h = blockIdx.y * 4 + wave;
  const int a0 = blockIdx.x * kKeysPerStep;
  int m0, n_rows;
  request_rows(p, b, m0, n_rows);
  if (h >= p.H) return;
  const float c = p.scale_log2e;
  const int kvh = h / (p.H / p.H_kv);
  const char *k_base = p.k_cache + p.affix_slot0 * p.kv_slot_bytes + (int64_t)kvh * p.kv_head_bytes;

  vec16 kf[4][KS];  // keys past the affix repeat the last one; their columns are not stored
#pragma unroll
  for (int nt = 0; nt < 4; ++nt) {
    const int a = a0 + 16 * nt + li;
    load_rows<D>(kf[nt], k_base + (int64_t)(a < p.A ? a : p.A - 1) * p.kv_slot_bytes, lg);
  }
  float col[4][4] = {};
  auto fetch = [&](int r0, vec16 (&qf)[NR][KS], float (&st)[NR]) __attribute__((always_inline)) {
#pragma unroll
    for (int t = 0; t < NR; ++t) {
      const int r = r0 + 16 * t + li;
      load_rows<D>(qf[t], mask_query_row(p, m0, n_rows, r, h), lg);
      st[t] = p.stats[(int64_t)(m0 + (r < n_rows ? r : n_rows - 1)) * p.H + h];
    }
  };
  // one step on the 32 rows in `qf`, with the next 32 requested first (always: past the end the clamped rows are
  // re-read and ignored, which keeps the loop free of a branch the loads would wait at)
  auto step = [&](int r0, vec16 (&qf)[NR][KS], float (&st)[NR], vec16 (&qf_next)[NR][KS], float (&st_next)[NR])
      __attribute__((always_inline)) {
    fetch(r0 + 16 * NR, qf_next, st_next);
#pragma unroll
    for (int t = 0; t < NR; ++t) {
      // a row past the request's end was read from a clamped address: 2^-inf = 0 keeps it out of the sums (the
      // test sits here, not at the load, so that the prefetch is not waited for the moment it is issued)
      const float ref = r0 + 16 * t + li < n_rows ? st[t] : INFINITY;
      f32x4 sc[4];
#pragma unroll
      for (int nt = 0; nt < 4; ++nt) sc[nt] = f32x4{0, 0, 0, 0};
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)  // four independent accumulator chains between two steps of one chain
#pragma unroll
        for (int nt = 0; nt < 4; ++nt) sc[nt] = M::run(kf[nt][ks], qf[t][ks], sc[nt]);
#pragma unroll
      for (int nt = 0; nt < 4; ++nt)
#pragma unroll
        for (int i = 0; i < 4; ++i) col[nt][i] += __builtin_amdgcn_exp2f(__builtin_fmaf(sc[nt][i], c, -ref));
    }
  };
  vec16 q_a[NR][KS], q_b[NR][KS];
  float st_a[NR], st_b[NR];
  if (n_rows > 0) fetch(0, q_a, st_a);
  for (int r0 = 0; r0 < n_rows; r0 += 32 * NR) {
    step(r0, q_a, st_a, q_b, st_b);
    if (r0 + 16 * NR < n_rows) step(r0 + 16 * NR, q_b, st_b, q_a, st_a);
  }
  // sum over the 16 query columns (lanes li) of every key row
  float *dst = p.partial + ((int64_t)b * p.H + h) * p.A;
#pragma unroll
  for (int nt = 0; nt < 4; ++nt)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float v = row_sum16(col[nt][i]);
      const int a = a0 + 16 * nt + 4 * lg + i;
      if (li == 0 && a < p.A) dst[a] = v;
    }
}

// ---------------------------------------------------------------------------------------------------
// The same two passes for head dims of 64, 128 and 256 with the streamed operand staged through LDS.
// In the kernels above every wave pulls the streamed rows (keys in the statistics pass, queries in the
// column pass) from L2 in operand layout, 64 bytes of a row per four lanes: the workgroup's four waves ask
// for the same or neighbouring rows four times over and the vector memory path, not the matrix core, sets
// the pace.  Here the four waves of a workgroup share one stream: the copy engine writes each 32-row tile
// into LDS once (whole rows, 16 bytes per lane, two buffers in turn) and all four waves read their
// fragments from there.  Rows are laid out with the 16-byte chunks of row r XOR-ed by r, so that the 16
// lanes reading one chunk column of 16 different rows hit 16 different bank groups.
constexpr int kStageRows = 32;  // query rows per LDS tile of the column pass
constexpr int kStageKeys = 64;  // keys per LDS tile of the statistics pass

template <int D, int ROWS>
struct StageGeometry {
  static constexpr int kChunks = D / 8;                   // 16-byte chunks per row (a power of two)
  static constexpr int kTileBytes = ROWS * D * 2;
  static constexpr int kCopiesPerWave = ROWS * D / 2048;  // 1 KiB wave copies per tile, split over four waves
  // chunk `c` of tile row `row` lives at this byte offset of the tile
  static __device__ __forceinline__ int offset(int row, int c) { return row * (D * 2) + ((c ^ (row & (kChunks - 1))) << 4); }
};

// Fragment of tile rows 16*t + li from LDS, in the layout load_rows() produces from global memory.
template <int D>
__device__ __forceinline__ void load_rows_lds(vec16 (&f)[D / 32], const char *tile, int t, int li, int lg) {
  using G = StageGeometry<D, 16>;  // the offset of a chunk does not depend on the tile height
#pragma unroll
  for (int ks = 0; ks < D / 32; ++ks) f[ks] = *(const vec16 *)(tile + G::offset(16 * t + li, 4 * ks + lg));
}

// Make the compiler finish a register-resident fragment's loads here.  Left alone it waits where the fragment is
// first used, inside the streaming loop, with a count that knows nothing of the LDS copies in flight there: a
// wait for "everything I issued" then also drains the copy of the next tile, every step.
__device__ __forceinline__ void settle(const vec16 &v) {
  asm volatile("" ::"v"(v.w[0]), "v"(v.w[1]), "v"(v.w[2]), "v"(v.w[3]));
}

// One workgroup per (request, head, 256 mask rows): wave w keeps rows 64*w .. 64*w + 63 in registers, the
// affix keys stream through LDS 32 at a time.  Same arithmetic and the same statistic as importance_stats_kernel.
template <int DTYPE, int D>
__global__ __launch_bounds__(256) void importance_stats_lds_kernel(ImportanceParams p) {
  constexpr int NQ = kRowTilesPerWave, KS = D / 32, NT = 2;  // key tiles scored together (a 64-key LDS tile: two rounds)
  using M = Mma<DTYPE>;
  using G = StageGeometry<D, kStageKeys>;
  __shared__ __attribute__((aligned(1024))) char tiles[2][G::kTileBytes];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int li = lane & 15, lg = lane >> 4;
  const int groups = (p.max_row_tiles + 4 * NQ - 1) / (4 * NQ);
  const int b = blockIdx.x / groups, rg = blockIdx.x % groups;
  const int h = blockIdx.y;
  int m0, n_rows;
  request_rows(p, b, m0, n_rows);
  if (rg * 4 * NQ * 16 >= n_rows) return;  // the whole workgroup: nothing to score
  const int row0 = (rg * 4 + wave) * NQ * 16;
  const bool live = row0 < n_rows;  // a wave past the request's rows still copies and synchronises
  const int kvh = h / (p.H / p.H_kv);
  const float c = p.scale_log2e;

  vec16 qf[NQ][KS];
#pragma unroll
  for (int qt = 0; qt < NQ; ++qt) load_rows<D>(qf[qt], mask_query_row(p, m0, n_rows, row0 + 16 * qt + li, h), lg);
#pragma unroll
  for (int qt = 0; qt < NQ; ++qt)
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) settle(qf[qt][ks]);

  // this lane's share of a tile copy: chunk slot `lane` of the 1 KiB piece (wave, j) holds which row and chunk?
  const char *k_base = p.k_cache + p.affix_slot0 * p.kv_slot_bytes + (int64_t)kvh * p.kv_head_bytes;
  int copy_row[G::kCopiesPerWave], copy_off[G::kCopiesPerWave];
#pragma unroll
  for (int j = 0; j < G::kCopiesPerWave; ++j) {
    const int slot = (wave * G::kCopiesPerWave + j) * 64 + lane;
    copy_row[j] = slot / G::kChunks;
    copy_off[j] = ((slot % G::kChunks) ^ (copy_row[j] & (G::kChunks - 1))) << 4;
  }
  auto issue = [&](int a0, int buf) __attribute__((always_inline)) {
#pragma unroll
    for (int j = 0; j < G::kCopiesPerWave; ++j) {
      const int a = a0 + copy_row[j];
      lds_dma16(k_base + (int64_t)(a < p.A ? a : p.A - 1) * p.kv_slot_bytes + copy_off[j],
                tiles[buf] + (wave * G::kCopiesPerWave + j) * 1024);
    }
  };

  float m_run[NQ], l_run[NQ];
#pragma unroll
  for (int qt = 0; qt < NQ; ++qt) { m_run[qt] = -INFINITY; l_run[qt] = 0.0f; }
  issue(0, 0);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  for (int t0 = 0, it = 0; t0 < p.A; t0 += kStageKeys, ++it) {
    issue(t0 + kStageKeys, (it + 1) & 1);  // always: past the end the last key is re-read and ignored
    if (live) {
      const char *tile = tiles[it & 1];
#pragma unroll
     for (int half = 0; half < kStageKeys / (16 * NT); ++half) {
      const int a0 = t0 + 16 * NT * half;
      if (a0 >= p.A) break;  // wave-uniform
      const bool tail = a0 + 16 * NT > p.A;
      vec16 kf[NT][KS];
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) load_rows_lds<D>(kf[nt], tile, NT * half + nt, li, lg);
#pragma unroll
      for (int qp = 0; qp < NQ; qp += 2) {
        f32x4 sc[2][NT];
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
          for (int nt = 0; nt < NT; ++nt) sc[u][nt] = f32x4{0, 0, 0, 0};
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
#pragma unroll
          for (int u = 0; u < 2; ++u)
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) sc[u][nt] = M::run(kf[nt][ks], qf[qp + u][ks], sc[u][nt]);
#pragma unroll
        for (int u = 0; u < 2; ++u) {
          const int qt = qp + u;
          if (tail) {
#pragma unroll
            for (int nt = 0; nt < NT; ++nt)
#pragma unroll
              for (int i = 0; i < 4; ++i)
                if (a0 + 16 * nt + 4 * lg + i >= p.A) sc[u][nt][i] = -INFINITY;
          }
          float mx = -INFINITY;
#pragma unroll
          for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int i = 0; i < 4; ++i) mx = fmaxf(mx, sc[u][nt][i]);
          mx = fmaxf(mx, __shfl_xor(mx, 16));
          mx = fmaxf(mx, __shfl_xor(mx, 32));
          const float m_new = fmaxf(m_run[qt], mx * c);
          float add = 0.0f;
#pragma unroll
          for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int i = 0; i < 4; ++i) add += __builtin_amdgcn_exp2f(__builtin_fmaf(sc[u][nt][i], c, -m_new));
          l_run[qt] = l_run[qt] * __builtin_amdgcn_exp2f(m_run[qt] - m_new) + add;
          m_run[qt] = m_new;
        }
      }
     }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the next tile has landed ...
    __syncthreads();                                    // ... and everybody is done with this one
  }
  if (!live) return;
#pragma unroll
  for (int qt = 0; qt < NQ; ++qt) {
    float l = l_run[qt];
    l += __shfl_xor(l, 16);
    l += __shfl_xor(l, 32);
    const int r = row0 + 16 * qt + li;
    if (lg == 0 && r < n_rows) {
      const int64_t src_row = p.mask_rows[m0 + r];
      const bool present = src_row >= 0 && src_row < p.total_q;
      p.stats[(int64_t)(m0 + r) * p.H + h] = present ? m_run[qt] + __builtin_amdgcn_logf(l) : INFINITY;
    }
  }
}

// One workgroup per (request, head, 256 affix keys): wave w keeps keys 64*w .. 64*w + 63 of the block in
// registers, the request's mask rows stream through LDS 32 at a time.  Same arithmetic as importance_colsum_kernel.
template <int DTYPE, int D>
__global__ __launch_bounds__(256) void importance_colsum_lds_kernel(ImportanceParams p) {
  constexpr int KS = D / 32, NR = kStageRows / 16;
  using M = Mma<DTYPE>;
  using G = StageGeometry<D, kStageRows>;
  __shared__ __attribute__((aligned(1024))) char tiles[2][G::kTileBytes];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int li = lane & 15, lg = lane >> 4;
  const int b = blockIdx.z;
  const int h = blockIdx.y;
  const int a0 = blockIdx.x * (4 * kKeysPerStep) + wave * kKeysPerStep;
  int m0, n_rows;
  request_rows(p, b, m0, n_rows);
  const bool live = a0 < p.A;  // a wave past the affix still copies and synchronises
  if (n_rows <= 0) {          // the whole workgroup: a request without mask rows has all-zero sums
    float *zero = p.partial + ((int64_t)b * p.H + h) * p.A;
    if (a0 + lane < p.A) zero[a0 + lane] = 0.0f;
    return;
  }
  const float c = p.scale_log2e;
  const int kvh = h / (p.H / p.H_kv);
  const char *k_base = p.k_cache + p.affix_slot0 * p.kv_slot_bytes + (int64_t)kvh * p.kv_head_bytes;

  vec16 kf[4][KS];
#pragma unroll
  for (int nt = 0; nt < 4; ++nt) {
    const int a = a0 + 16 * nt + li;
    load_rows<D>(kf[nt], k_base + (int64_t)(a < p.A ? a : p.A - 1) * p.kv_slot_bytes, lg);
  }
#pragma unroll
  for (int nt = 0; nt < 4; ++nt)
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) settle(kf[nt][ks]);
  int copy_row[G::kCopiesPerWave], copy_off[G::kCopiesPerWave];
#pragma unroll
  for (int j = 0; j < G::kCopiesPerWave; ++j) {
    const int slot = (wave * G::kCopiesPerWave + j) * 64 + lane;
    copy_row[j] = slot / G::kChunks;
    copy_off[j] = ((slot % G::kChunks) ^ (copy_row[j] & (G::kChunks - 1))) << 4;
  }
  auto issue = [&](int r0, int buf) __attribute__((always_inline)) {
#pragma unroll
    for (int j = 0; j < G::kCopiesPerWave; ++j)
      lds_dma16(mask_query_row(p, m0, n_rows, r0 + copy_row[j], h) + copy_off[j],
                tiles[buf] + (wave * G::kCopiesPerWave + j) * 1024);
  };
  auto statistic = [&](int r0, float (&st)[NR]) __attribute__((always_inline)) {
#pragma unroll
    for (int t = 0; t < NR; ++t) {
      const int r = r0 + 16 * t + li;
      st[t] = p.stats[(int64_t)(m0 + (r < n_rows ? r : n_rows - 1)) * p.H + h];
    }
  };
  float col[4][4] = {};
  float st_cur[NR], st_next[NR];
  statistic(0, st_cur);
  issue(0, 0);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  for (int r0 = 0, it = 0; r0 < n_rows; r0 += kStageRows, ++it) {
    statistic(r0 + kStageRows, st_next);       // ordinary loads first, then the copies behind them
    issue(r0 + kStageRows, (it + 1) & 1);      // always: past the end the last row is re-read and ignored
    if (live) {
      const char *tile = tiles[it & 1];
#pragma unroll
      for (int t = 0; t < NR; ++t) {
        const float ref = r0 + 16 * t + li < n_rows ? st_cur[t] : INFINITY;  // 2^-inf = 0 for rows past the end
        vec16 qf[KS];
        load_rows_lds<D>(qf, tile, t, li, lg);
        f32x4 sc[4];
#pragma unroll
        for (int nt = 0; nt < 4; ++nt) sc[nt] = f32x4{0, 0, 0, 0};
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
#pragma unroll
          for (int nt = 0; nt < 4; ++nt) sc[nt] = M::run(kf[nt][ks], qf[ks], sc[nt]);
#pragma unroll
        for (int nt = 0; nt < 4; ++nt)
#pragma unroll
          for (int i = 0; i < 4; ++i) col[nt][i] += __builtin_amdgcn_exp2f(__builtin_fmaf(sc[nt][i], c, -ref));
      }
    }
#pragma unroll
    for (int t = 0; t < NR; ++t) st_cur[t] = st_next[t];
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the next tile has landed ...
    __syncthreads();                                    // ... and everybody is done with this one
  }
  if (!live) return;
  float *dst = p.partial + ((int64_t)b * p.H + h) * p.A;
#pragma unroll
  for (int nt = 0; nt < 4; ++nt)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float v = row_sum16(col[nt][i]);
      const int a = a0 + 16 * nt + 4 * lg + i;
      if (li == 0 && a < p.A) dst[a] = v;
    }
}

// importance[b, a] += sum over heads of partial[b, h, a], in a fixed order: four lanes take every fourth head
// each (their loads all in flight together), then the four shares are added in lane order.
__global__ __launch_bounds__(256) void importance_reduce_kernel(ImportanceParams p) {
  __shared__ float share[4][64];
  const int a = blockIdx.x * 64 + (threadIdx.x & 63);
  const int part = threadIdx.x >> 6;
  const int b = blockIdx.y;
  float acc = 0.0f;
  if (a < p.A) {
    const float *src = p.partial + (int64_t)b * p.H * p.A + a;
#pragma unroll 8
    for (int h = part; h < p.H; h += 4) acc += src[(int64_t)h * p.A];
  }
  share[part][threadIdx.x & 63] = acc;
  __syncthreads();
  if (part == 0 && a < p.A) {
    const int j = threadIdx.x;
    p.importance[(int64_t)b * p.imp_stride + a] += ((share[0][j] + share[1][j]) + share[2][j]) + share[3][j];
  }
}

}  // namespace acache

using namespace acache;

static int64_t stats_bytes(int64_t total_mask_rows, int32_t H) {
  return (total_mask_rows * H * (int64_t)sizeof(float) + 15) / 16 * 16;
}

static int64_t partial_bytes(int32_t B, int32_t H, int32_t affix_len) {
  return ((int64_t)B * H * affix_len * (int64_t)sizeof(float) + 15) / 16 * 16;
}

extern "C" int64_t acache_affix_importance_workspace_bytes(int64_t total_mask_rows, int32_t B, int32_t H,
                                                           int32_t H_kv, int32_t D, int32_t affix_len,
                                                           int32_t relocated) {
  if (total_mask_rows < 0 || B < 0 || H < 0 || H_kv < 0 || D < 0 || affix_len < 0) return 0;
  (void)H_kv;
  (void)relocated;  // the packed copy of the mask queries (2-byte elements) is made with and without relocation
  return stats_bytes(total_mask_rows, H) + partial_bytes(B, H, affix_len) + total_mask_rows * H * D * 2;
}

// Argument checks and the launches; `workspace` is caller memory or this library's file-scope scratch.
static int importance_launch(
    float *importance, const void *q, const void *k_cache, const int32_t *mask_rows, const int32_t *cu_mask,
    const int32_t *affix_shifts, const float *rope_cos, const float *rope_sin, int32_t rope_rows, float scale,
    int32_t affix_len, int64_t affix_slot0, int32_t B, int64_t total_q, int64_t total_mask_rows, int32_t max_mask_rows,
    int32_t H,
    int32_t H_kv, int32_t D, int32_t dtype, int64_t num_slots, int64_t importance_stride, int64_t q_token_stride,
    int64_t q_head_stride, int64_t kv_slot_stride, int64_t kv_head_stride, void *workspace, int64_t workspace_bytes,
    void *stream) {
  if (dtype != ACACHE_BF16 && dtype != ACACHE_F16)
    return fail(ACACHE_E_DTYPE, "affix_importance: dtype %d not supported (bf16 or f16)", dtype);
  if (D < 16 || D > 256 || D % 16 != 0)
    return fail(ACACHE_E_SHAPE, "affix_importance: head_dim %d not supported (a multiple of 16 up to 256)", D);
  if (B < 0 || affix_len < 0 || total_mask_rows < 0 || max_mask_rows < 0 || H <= 0 || H_kv <= 0 || H % H_kv)
    return fail(ACACHE_E_SHAPE, "affix_importance: bad sizes (B %d, A %d, H %d, H_kv %d)", B, affix_len, H, H_kv);
  if (B == 0 || affix_len == 0 || total_mask_rows == 0 || max_mask_rows == 0) return 0;
  if (total_q <= 0) return fail(ACACHE_E_SHAPE, "affix_importance: %lld mask rows but q has %lld rows",
                                (long long)total_mask_rows, (long long)total_q);
  if (!importance || !q || !k_cache || !mask_rows || !cu_mask || !workspace)
    return fail(ACACHE_E_NULL, "affix_importance: NULL pointer");
  if (affix_shifts && (!rope_cos || !rope_sin || rope_rows <= 0))
    return fail(ACACHE_E_MODE, "affix_importance: shifts given without RoPE tables");
  if (!(scale > 0.0f)) return fail(ACACHE_E_RANGE, "affix_importance: scale must be positive");
  if (affix_slot0 < 0 || affix_slot0 + affix_len > num_slots)
    return fail(ACACHE_E_RANGE, "affix_importance: affix slots [%lld, %lld) outside %lld slots", (long long)affix_slot0,
                (long long)(affix_slot0 + affix_len), (long long)num_slots);
  if (importance_stride < affix_len) return fail(ACACHE_E_SHAPE, "affix_importance: importance stride < affix_len");
  if (total_mask_rows * H * D * 2 >= ((int64_t)1 << 32))
    return fail(ACACHE_E_SHAPE, "affix_importance: %lld mask rows x %d heads x %d: the packed query copy must stay under 4 GiB",
                (long long)total_mask_rows, H, D);
  if (workspace_bytes < acache_affix_importance_workspace_bytes(total_mask_rows, B, H, H_kv, D, affix_len, affix_shifts != nullptr))
    return fail(ACACHE_E_SHAPE, "affix_importance: workspace of %lld bytes, %lld needed", (long long)workspace_bytes,
                (long long)acache_affix_importance_workspace_bytes(total_mask_rows, B, H, H_kv, D, affix_len, affix_shifts != nullptr));
  if (!aligned16(q) || !aligned16(k_cache) || !aligned16(workspace) || (rope_cos && !aligned16(rope_cos)) ||
      (rope_sin && !aligned16(rope_sin)) || (q_token_stride * 2) % 16 || (q_head_stride * 2) % 16 ||
      (kv_slot_stride * 2) % 16 || (kv_head_stride * 2) % 16)
    return fail(ACACHE_E_ALIGN, "affix_importance: pointers and strides must be 16-byte aligned");
  ImportanceParams p;
  p.importance = importance; p.q = (const char *)q; p.k_cache = (const char *)k_cache;
  p.mask_rows = mask_rows; p.cu_mask = cu_mask; p.shifts = affix_shifts;
  p.cos_tab = rope_cos; p.sin_tab = rope_sin; p.stats = (float *)workspace;
  p.partial = (float *)((char *)workspace + stats_bytes(total_mask_rows, H));
  p.q_rot = (char *)workspace + stats_bytes(total_mask_rows, H) + partial_bytes(B, H, affix_len);
  p.total_q = total_q;
  p.imp_stride = importance_stride;
  p.q_token_bytes = q_token_stride * 2; p.q_head_bytes = q_head_stride * 2;
  p.kv_slot_bytes = kv_slot_stride * 2; p.kv_head_bytes = kv_head_stride * 2;
  p.affix_slot0 = affix_slot0;
  p.scale_log2e = scale * 1.4426950408889634f;
  p.A = affix_len; p.B = B; p.H = H; p.H_kv = H_kv; p.rope_rows = rope_rows; p.D = D;
  p.max_row_tiles = (max_mask_rows + 15) / 16;
  p.total_mask_rows = (int32_t)total_mask_rows;
  p.max_mask_rows = max_mask_rows;
  hipStream_t s = (hipStream_t)stream;
  const int lanes_per_row = D * 2 / 32;
  const dim3 grid0((unsigned)(((int64_t)max_mask_rows * H * lanes_per_row + 255) / 256), (unsigned)B);
  const int row_groups = (p.max_row_tiles + kRowTilesPerWave - 1) / kRowTilesPerWave;
  const dim3 grid1((unsigned)((int64_t)B * row_groups), (unsigned)((H + 3) / 4));
  const dim3 grid2((unsigned)((affix_len + kKeysPerStep - 1) / kKeysPerStep), (unsigned)((H + 3) / 4), (unsigned)B);
  const dim3 grid3((unsigned)((affix_len + 63) / 64), (unsigned)B);
  // the LDS-staged pair: a workgroup per (request, head, 256 mask rows) and per (request, head, 256 affix keys)
  const int row_groups_staged = (p.max_row_tiles + 4 * kRowTilesPerWave - 1) / (4 * kRowTilesPerWave);
  const dim3 grid1s((unsigned)((int64_t)B * row_groups_staged), (unsigned)H);
  const dim3 grid2s((unsigned)((affix_len + 4 * kKeysPerStep - 1) / (4 * kKeysPerStep)), (unsigned)H, (unsigned)B);
#define ACACHE_CASE(DT, HD)                                                                       \
  if (dtype == DT && D == HD) {                                                                   \
    hipLaunchKernelGGL((importance_rotate_kernel<DT>), grid0, dim3(256), 0, s, p);                \
    const int rc0 = launch_status("importance_rotate_kernel");                                    \
    if (rc0) return rc0;                                                                          \
    if constexpr (HD == 64 || HD == 128 || HD == 256) {                                           \
      hipLaunchKernelGGL((importance_stats_lds_kernel<DT, HD>), grid1s, dim3(256), 0, s, p);      \
      const int rc = launch_status("importance_stats_lds_kernel");                                \
      if (rc) return rc;                                                                          \
      hipLaunchKernelGGL((importance_colsum_lds_kernel<DT, HD>), grid2s, dim3(256), 0, s, p);     \
      const int rc2 = launch_status("importance_colsum_lds_kernel");                              \
      if (rc2) return rc2;                                                                        \
    } else {                                                                                      \
      hipLaunchKernelGGL((importance_stats_kernel<DT, HD>), grid1, dim3(256), 0, s, p);           \
      const int rc = launch_status("importance_stats_kernel");                                    \
      if (rc) return rc;                                                                          \
      hipLaunchKernelGGL((importance_colsum_kernel<DT, HD>), grid2, dim3(256), 0, s, p);          \
      const int rc2 = launch_status("importance_colsum_kernel");                                  \
      if (rc2) return rc2;                                                                        \
    }                                                                                             \
    hipLaunchKernelGGL(importance_reduce_kernel, grid3, dim3(256), 0, s, p);                      \
    return launch_status("importance_reduce_kernel");                                             \
  }
#define ACACHE_DIMS(DT)                                                                             \
  ACACHE_CASE(DT, 128) ACACHE_CASE(DT, 64) ACACHE_CASE(DT, 16) ACACHE_CASE(DT, 32) ACACHE_CASE(DT, 48)   \
  ACACHE_CASE(DT, 80) ACACHE_CASE(DT, 96) ACACHE_CASE(DT, 112) ACACHE_CASE(DT, 144) ACACHE_CASE(DT, 160) \
  ACACHE_CASE(DT, 176) ACACHE_CASE(DT, 192) ACACHE_CASE(DT, 208) ACACHE_CASE(DT, 224) ACACHE_CASE(DT, 240) \
  ACACHE_CASE(DT, 256)
  ACACHE_DIMS(ACACHE_BF16)
  ACACHE_DIMS(ACACHE_F16)
#undef ACACHE_DIMS
#undef ACACHE_CASE
  return fail(ACACHE_E_SHAPE, "affix_importance: unsupported dtype / head_dim");
}

extern "C" int acache_affix_importance(
    float *importance, const void *q, const void *k_cache, const int32_t *mask_rows, const int32_t *cu_mask,
    const int32_t *affix_shifts, const float *rope_cos, const float *rope_sin, int32_t rope_rows, float scale,
    int32_t affix_len, int64_t affix_slot0, int32_t B, int64_t total_q, int64_t total_mask_rows, int32_t max_mask_rows,
    int32_t H,
    int32_t H_kv, int32_t D, int32_t dtype, int64_t num_slots, int64_t importance_stride, int64_t q_token_stride,
    int64_t q_head_stride, int64_t kv_slot_stride, int64_t kv_head_stride, void *workspace, int64_t workspace_bytes,
    void *stream) {
  return importance_launch(importance, q, k_cache, mask_rows, cu_mask, affix_shifts, rope_cos, rope_sin, rope_rows, scale,
                           affix_len, affix_slot0, B, total_q, total_mask_rows, max_mask_rows, H, H_kv, D, dtype, num_slots,
                           importance_stride, q_token_stride, q_head_stride, kv_slot_stride, kv_head_stride, workspace,
                           workspace_bytes, stream);
}

// ---------------------------------------------------------------------------------------------------
// The same call for callers that cannot allocate device memory (code under HIP graph capture, serving
// loops, harnesses that forbid hipMalloc): the row statistics, per-head partial sums and counter-rotated queries
// live in a file-scope device array instead of a caller workspace.  Every GPU the library runs on holds
// its own copy of the array at its own address until the process ends; the address is looked up once per
// device and only that pointer is ever handed to kernels.  Nothing in the array has to start at zero:
// every word a launch reads was written by an earlier launch of the same call.
static __device__ __align__(256) unsigned char scratch[ACACHE_IMPORTANCE_SCRATCH_BYTES];

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void *g_scratch_ptr[kMaxDevices] = {};

int scratch_of_current_device(void **out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return fail((int)e, "affix_importance_noalloc: hipGetDevice: %s", hipGetErrorString(e));
  if (dev < 0 || dev >= kMaxDevices)
    return fail(ACACHE_E_RANGE, "affix_importance_noalloc: device %d outside the %d devices supported", dev, kMaxDevices);
  std::lock_guard<std::mutex> guard(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void *ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !ptr)
      return fail(e != hipSuccess ? (int)e : ACACHE_E_NULL, "affix_importance_noalloc: hipGetSymbolAddress: %s",
                  hipGetErrorString(e));
    g_scratch_ptr[dev] = ptr;
  }
  *out = g_scratch_ptr[dev];
  return 0;
}
}  // namespace

extern "C" int64_t acache_affix_importance_noalloc_max_bytes(void) { return ACACHE_IMPORTANCE_SCRATCH_BYTES; }

extern "C" int acache_affix_importance_noalloc(
    float *importance, const void *q, const void *k_cache, const int32_t *mask_rows, const int32_t *cu_mask,
    const int32_t *affix_shifts, const float *rope_cos, const float *rope_sin, int32_t rope_rows, float scale,
    int32_t affix_len, int64_t affix_slot0, int32_t B, int64_t total_q, int64_t total_mask_rows, int32_t max_mask_rows,
    int32_t H,
    int32_t H_kv, int32_t D, int32_t dtype, int64_t num_slots, int64_t importance_stride, int64_t q_token_stride,
    int64_t q_head_stride, int64_t kv_slot_stride, int64_t kv_head_stride, void *stream) {
  const int64_t need =
      acache_affix_importance_workspace_bytes(total_mask_rows, B, H, H_kv, D, affix_len, affix_shifts != nullptr);
  if (need > (int64_t)ACACHE_IMPORTANCE_SCRATCH_BYTES)
    return fail(ACACHE_E_SHAPE,
                "affix_importance_noalloc: this call needs %lld bytes of scratch, the built-in buffer holds %lld; "
                "use acache_affix_importance with a caller workspace",
                (long long)need, (long long)ACACHE_IMPORTANCE_SCRATCH_BYTES);
  void *ws = nullptr;
  const int rc = scratch_of_current_device(&ws);
  if (rc) return rc;
  return importance_launch(importance, q, k_cache, mask_rows, cu_mask, affix_shifts, rope_cos, rope_sin, rope_rows, scale,
                           affix_len, affix_slot0, B, total_q, total_mask_rows, max_mask_rows, H, H_kv, D, dtype, num_slots,
                           importance_stride, q_token_stride, q_head_stride, kv_slot_stride, kv_head_stride, ws,
                           ACACHE_IMPORTANCE_SCRATCH_BYTES, stream);
}
