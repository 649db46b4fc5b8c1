// Bidirectional varlen attention over slot-mapped K/V on gfx950 MFMA.
//
// Work decomposition
//   workgroup = 4 waves; each wave owns WQ = 16*NQ16 consecutive queries of one
//   (request, head); the workgroup owns BM = 4*WQ queries and walks the request's
//   keys in tiles of BN = 64, staged through LDS and shared by the 4 waves.
//
// MFMA formulation (v_mfma_f32_16x16x32, 64-wide wavefronts)
//   S^T = K Q^T   : A = K tile rows from LDS, B = Q (registers)
//   O^T = V^T P^T : A = V^T from LDS, B = P^T, which is exactly the accumulator
//                   layout of S^T after a bf16 pack — probabilities never leave
//                   registers.
//   In both products a lane owns ONE query column, so the running maximum and the
//   rescale factor are per-lane scalars; the softmax denominator is one more
//   MFMA row block (V^T rows of ones).
//
// Two kernels:
//   varlen_attn_unit_kernel (head_dim 64 and 128, all three relocation modes): K/V rows are copied
//     global -> LDS directly through the slot map into a two-deep ring, swizzled by permuting the
//     global side of the copy; V stays row-major and is read with the LDS transpose read.  Scores are
//     scaled in fp32 inside the softmax (one fused multiply-add per score in front of exp2), as the
//     reference scales the fp32 product.
//     Key-side relocation re-rotates the shared rows of a tile in LDS once it has landed.
//   varlen_attn_kernel (any other head_dim): rows are staged through registers, re-rotated there in
//     key-side mode, and V is transposed on the way into LDS; scores are scaled in the softmax.
// Within a kernel all modes share the softmax steps, so key-side relocation rounds exactly like
// attention over a materialised copy.  HBM traffic per call: K and V rows once per (request, kv head)
// when query tiles of one head share an L2 (block indices are mapped so that they land on the same
// XCD), Q once, O once.
#include <stdlib.h>
#include "attn_common.h"

namespace acache {

// Register-staged kernel: every mode at a head_dim other than 64 / 128.
//
// RAGGED = true is the any-head_dim variant: D is then the padded width (a multiple of 32) and the real
// head_dim (a multiple of 16, at most D) comes in p.head_dim.  Rows are laid out in LDS at their real
// width, the padding columns are zeroed once and never written again, and every loop over k-slabs and
// d tiles skips the ones past the real width with a wave-uniform test.  Same arithmetic per element.
template <int DTYPE, int D, int NQ16, int MODE, bool RAGGED = false>
__global__ __launch_bounds__(256, RAGGED ? 1 : 2) void varlen_attn_kernel(AttnParams p) {
  constexpr int BN = 64;
  constexpr int WQ = 16 * NQ16;
  constexpr int BM = 4 * WQ;
  constexpr int KS = D / 32;            // k-slabs of the QK^T product
  constexpr int NT = BN / 16;           // 16-row key tiles per BN
  constexpr int DT = D / 16;            // 16-row d tiles of O^T
  constexpr int NS = BN / 32;           // 32-key slabs of the PV product
  constexpr int ROW_BYTES = D * 2;
  constexpr int CH = ROW_BYTES / 16;    // 16-byte chunks per row
  constexpr int PP = CH / 2;            // chunk pairs per row (K loader)
  constexpr int K_PAIRS = BN * PP;      // one thread per (row, chunk pair) and pass
  constexpr int K_PASSES = (K_PAIRS + 255) / 256;
  // the padded variant swizzles the chunks of a K row instead of padding the pitch (64 KiB of LDS at D = 256)
  constexpr int KPITCH = RAGGED ? ROW_BYTES : ROW_BYTES + 16;
  constexpr int V_ITEMS = CH * (BN / 4);  // one thread per (chunk, 4-row group) and pass
  constexpr int V_PASSES = (V_ITEMS + 255) / 256;
  constexpr int VPITCH = BN * 2;            // bytes per V^T row (swizzled, unpadded)
  using M = Mma<DTYPE>;

  __shared__ __attribute__((aligned(16))) char lds_k[BN * KPITCH];
  __shared__ __attribute__((aligned(16))) char lds_v[D * VPITCH];

  const int d_real = RAGGED ? p.head_dim : D;
  const int ch_real = d_real / 8;       // 16-byte chunks of a real row
  const int pp_real = ch_real / 2;      // the rotate-half partner of chunk c is chunk c + pp_real
  // position of chunk c of K row r inside its LDS row
  auto kpos = [](int r, int c) __attribute__((always_inline)) { return RAGGED ? (c ^ (r & 15)) : c; };

  // ---- which (request, query tile, head) is this workgroup? -----------------
  const int per_xcd = gridDim.x >> 3;
  const int w = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
  const int group = p.H / p.H_kv;
  if (w >= p.num_tiles * p.H) return;
  const int hg = w % group;
  int tile = (w / group) % p.num_tiles;
  const int kvh = w / (group * p.num_tiles);
  const int head = kvh * group + hg;
  int b = 0, q_begin = 0, q_len = 0;
  {
    int tile_in_request = 0;
    if (!locate_query_tile(p.cu_q, p.B, BM, tile, b, q_begin, q_len, tile_in_request)) return;
    tile = tile_in_request;
  }

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int li = lane & 15, lg = lane >> 4;
  const int kv_begin = p.cu_k[b];
  const int kv_len = p.cu_k[b + 1] - kv_begin;
  const int q_tile0 = tile * BM;                  // first query row of the workgroup
  const int q_wave0 = q_tile0 + wave * WQ;        // first query row of this wave
  int nq_valid = (q_len - q_wave0 + 15) / 16;     // live 16-row query tiles of this wave
  nq_valid = nq_valid < 0 ? 0 : (nq_valid > NQ16 ? NQ16 : nq_valid);

  char *out_base = p.out + (int64_t)q_begin * p.o_token_bytes + (int64_t)head * p.o_head_bytes;

  if (kv_len <= 0) {  // no keys: defined output (zeros)
    for (int r = tid / CH; r < BM; r += 256 / CH) {
      const int qr = q_tile0 + r;
      if (qr < q_len && tid % CH < ch_real)
        store16(out_base + (int64_t)qr * p.o_token_bytes + (tid % CH) * 16, vec16{{0, 0, 0, 0}});
    }
    return;
  }

  int shared_len = 0, shift = 0;
  if (MODE == MODE_QUERY_SIDE) {
    shared_len = p.shared_kv_lens[b];
    shared_len = shared_len < 0 ? 0 : (shared_len > kv_len ? kv_len : shared_len);
    shift = p.affix_shifts[b];
    if (shift < 0 || shift >= p.rope_rows) shift = 0;  // out-of-table shift: leave unrotated
  }

  // ---- Q fragments (B operand): lane holds Q[query li][32*ks + 8*lg .. +8] ---
  vec16 qf[NQ16][KS];
  vec16 qs[NQ16][KS];  // query-side mode: rotated copy scored against the shared keys
  const char *q_base = p.q + (int64_t)q_begin * p.q_token_bytes + (int64_t)head * p.q_head_bytes;
#pragma unroll
  for (int qt = 0; qt < NQ16; ++qt) {
    const int qr = q_wave0 + qt * 16 + li;
    const bool live = qr < q_len;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      qf[qt][ks] = live && 32 * ks + 8 * lg < d_real
                       ? load16(q_base + (int64_t)qr * p.q_token_bytes + (32 * ks + 8 * lg) * 2)
                       : vec16{{0, 0, 0, 0}};
    }
    if (MODE == MODE_QUERY_SIDE && !RAGGED) {
      const float *cr = p.cos_tab + (int64_t)shift * D;
      const float *sr = p.sin_tab + (int64_t)shift * D;
#pragma unroll
      for (int ks = 0; ks < KS / 2; ++ks) {  // partner of d is d + D/2: slab ks + KS/2, same lane
        vec16 lo = qf[qt][ks], hi = qf[qt][ks + KS / 2];
        if (shift != 0) rotate_pair<DTYPE, D>(lo, hi, cr, sr, 32 * ks + 8 * lg, -1.0f);
        qs[qt][ks] = lo;
        qs[qt][ks + KS / 2] = hi;
      }
    }
    if (MODE == MODE_QUERY_SIDE && RAGGED) {
      // the partner chunk (d +- head_dim/2) belongs to another lane here: fetch it, rotate the pair, keep our half
      const float *cr = p.cos_tab + (int64_t)shift * d_real;
      const float *sr = p.sin_tab + (int64_t)shift * d_real;
      const int half = d_real / 2;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const int d0 = 32 * ks + 8 * lg;
        qs[qt][ks] = qf[qt][ks];
        if (live && d0 < d_real && shift != 0) {
          const bool first = d0 < half;
          const int dl = first ? d0 : d0 - half;
          const vec16 other = load16(q_base + (int64_t)qr * p.q_token_bytes + (first ? d0 + half : dl) * 2);
          vec16 lo = first ? qf[qt][ks] : other, hi = first ? other : qf[qt][ks];
          rotate_pair_half<DTYPE>(lo, hi, cr, sr, dl, half, -1.0f);
          qs[qt][ks] = first ? lo : hi;
        }
      }
    }
  }

  // ---- loader state ------------------------------------------------------------
  // K: thread -> (row kr0 + pass * K_ROWS_PER_PASS, chunk pair kc / kc + pp_real)
  // V: thread -> (chunk vc, rows 4*vrg .. 4*vrg+3 with vrg = vrg0 + pass * V_GROUPS_PER_PASS)
  // row groups past the tile, and chunks past the real row width, stay idle
  static_assert(256 % PP == 0 && K_PAIRS % 256 == 0 && 256 % CH == 0, "the loaders want a power-of-two row width");
  constexpr int K_ROWS_PER_PASS = 256 / PP;
  constexpr int V_GROUPS_PER_PASS = 256 / CH;
  const int kr0 = tid / PP, kc = tid % PP;
  const int vc = tid % CH, vrg0 = tid / CH;
  const bool k_thread = !RAGGED || kc < pp_real;
  vec16 k_lo[K_PASSES], k_hi[K_PASSES], v_row[V_PASSES][4];
  const char *kc_base = p.k_cache + (int64_t)kvh * p.kv_head_bytes;
  const char *vc_base = p.v_cache + (int64_t)kvh * p.kv_head_bytes;
  auto v_live = [&](int vrg) __attribute__((always_inline)) {
    return (V_ITEMS % 256 == 0 || vrg < BN / 4) && (!RAGGED || vc < ch_real);
  };

  if (RAGGED) {  // the padding columns of both tiles are zero for the whole kernel
    for (int i = tid * 16; i < BN * KPITCH; i += 256 * 16) store16(lds_k + i, vec16{{0, 0, 0, 0}});
    for (int i = tid * 16; i < D * VPITCH; i += 256 * 16) store16(lds_v + i, vec16{{0, 0, 0, 0}});
    __syncthreads();
  }

  auto fetch = [&](int n0, int n_end) __attribute__((always_inline)) {
#pragma unroll
    for (int ps = 0; ps < K_PASSES; ++ps) {
      const int n = n0 + kr0 + ps * K_ROWS_PER_PASS;
      k_lo[ps] = vec16{{0, 0, 0, 0}};
      k_hi[ps] = k_lo[ps];
      if (k_thread && n < n_end) {
        const int64_t slot = p.slot_map[kv_begin + n];
        if (slot >= 0 && slot < p.num_slots) {
          const char *src = kc_base + slot * p.kv_slot_bytes + kc * 16;
          k_lo[ps] = load16(src);
          k_hi[ps] = load16(src + pp_real * 16);
          if (MODE == MODE_KEY_SIDE && slot < p.shared_prefix_len) {
            const int delta = n - (int)slot;
            const int ad = delta < 0 ? -delta : delta;
            if (delta != 0 && ad < p.rope_rows)
              rotate_pair_half<DTYPE>(k_lo[ps], k_hi[ps], p.cos_tab + (int64_t)ad * d_real,
                                      p.sin_tab + (int64_t)ad * d_real, kc * 8, d_real / 2,
                                      delta < 0 ? -1.0f : 1.0f);
          }
        }
      }
    }
#pragma unroll
    for (int ps = 0; ps < V_PASSES; ++ps) {
      const int vrg = vrg0 + ps * V_GROUPS_PER_PASS;
      if (v_live(vrg)) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int n = n0 + 4 * vrg + r;
          v_row[ps][r] = vec16{{0, 0, 0, 0}};
          if (n < n_end) {
            const int64_t slot = p.slot_map[kv_begin + n];
            if (slot >= 0 && slot < p.num_slots) v_row[ps][r] = load16(vc_base + slot * p.kv_slot_bytes + vc * 16);
          }
        }
      }
    }
  };

  auto stage = [&]() __attribute__((always_inline)) {
#pragma unroll
    for (int ps = 0; ps < K_PASSES; ++ps) {
      const int kr = kr0 + ps * K_ROWS_PER_PASS;
      if (k_thread) {
        char *dst = lds_k + kr * KPITCH;
        store16(dst + kpos(kr, kc) * 16, k_lo[ps]);
        store16(dst + kpos(kr, kc + pp_real) * 16, k_hi[ps]);
      }
    }
#pragma unroll
    for (int ps = 0; ps < V_PASSES; ++ps) {
      const int vrg = vrg0 + ps * V_GROUPS_PER_PASS;
      if (v_live(vrg)) {
        // 4 rows x 8 elements -> 8 columns x 4 keys; key n sits at position
        // 32*(n/32) + 8*((n%16)/4) + 4*((n%32)/16) + n%4 inside its V^T row, the
        // order in which the S^T accumulator hands probabilities to the PV product
        const int n4 = 4 * vrg;
        const int chunk = 4 * (n4 >> 5) + ((n4 & 15) >> 2);
        const int half = (n4 & 31) >> 4;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const int d = 8 * vc + j;
          const uint32_t w0 = v_row[ps][0].w[j >> 1], w1 = v_row[ps][1].w[j >> 1];
          const uint32_t w2 = v_row[ps][2].w[j >> 1], w3 = v_row[ps][3].w[j >> 1];
          uint2 val;
          if (j & 1) {
            val.x = (w0 >> 16) | (w1 & 0xffff0000u);
            val.y = (w2 >> 16) | (w3 & 0xffff0000u);
          } else {
            val.x = (w0 & 0xffffu) | (w1 << 16);
            val.y = (w2 & 0xffffu) | (w3 << 16);
          }
          const int swz = ((d >> 1) & 7) ^ ((d >> 4) & 7);
          *reinterpret_cast<uint2 *>(lds_v + d * VPITCH + ((chunk ^ swz) << 4) + (half << 3)) = val;
        }
      }
    }
  };

  // ---- running softmax state, one query column per lane -------------------------
  float m_run[NQ16];
  f32x4 o_acc[NQ16][DT], l_acc[NQ16];
  const uint32_t one2 = M::pack2(1.0f, 1.0f);
  const vec16 ones{{one2, one2, one2, one2}};
#pragma unroll
  for (int qt = 0; qt < NQ16; ++qt) {
    m_run[qt] = -INFINITY;
    l_acc[qt] = f32x4{0, 0, 0, 0};
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) o_acc[qt][dt] = f32x4{0, 0, 0, 0};
  }

  // tiles: first the shared range [0, shared_len) (query-side mode only), then the rest
  const int tiles_a = (shared_len + BN - 1) / BN;
  const int tiles_b = (kv_len - shared_len + BN - 1) / BN;
  const int n_tiles = tiles_a + tiles_b;

  int n0, n_end;
  { const TileRange tr = tile_range_of(0, tiles_a, shared_len, kv_len, BN); n0 = tr.n0; n_end = tr.n_end; }
  fetch(n0, n_end);

  const float c = p.scale_log2e;
  for (int t = 0; t < n_tiles; ++t) {
    { const TileRange tr = tile_range_of(t, tiles_a, shared_len, kv_len, BN); n0 = tr.n0; n_end = tr.n_end; }
    const int n_valid = n_end - n0;  // keys of this tile that exist (may exceed BN)
    const bool shared_tile = MODE == MODE_QUERY_SIDE && t < tiles_a;
    stage();
    __syncthreads();
    if (t + 1 < n_tiles) {
      int m0, m_end;
      { const TileRange tr = tile_range_of(t + 1, tiles_a, shared_len, kv_len, BN); m0 = tr.n0; m_end = tr.n_end; }
      fetch(m0, m_end);
    }

    if (nq_valid > 0) {  // waves past the end of the request only help with the loads
    // K fragments (A operand): lane holds K[16*nt + li][32*ks + 8*lg .. +8]
    f32x4 s_acc[NQ16][NT];
#pragma unroll
    for (int qt = 0; qt < NQ16; ++qt)
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) s_acc[qt][nt] = f32x4{0, 0, 0, 0};
    auto scores = [&](const vec16 (&qq)[NQ16][KS]) __attribute__((always_inline)) {
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) {
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
          if (RAGGED && 32 * ks >= d_real) continue;
          const vec16 kf = load16(lds_k + (16 * nt + li) * KPITCH + kpos(li, 4 * ks + lg) * 16);
#pragma unroll
          for (int qt = 0; qt < NQ16; ++qt)
            s_acc[qt][nt] = M::run(kf, qq[qt][ks], s_acc[qt][nt]);
        }
      }
    };
    if (MODE == MODE_QUERY_SIDE && shared_tile) scores(qs);
    else scores(qf);

    // online softmax; P^T packed straight into the B operand of the PV product
    vec16 pf[NQ16][NS];
    softmax_reference<NQ16, NQ16, NT, DT, true>(s_acc, m_run, l_acc, o_acc, c, n_valid, lg);
    static_assert(NS == 2, "two 32-key slabs per tile");
    softmax_probs_slab<M, 0, NQ16>(s_acc, m_run, l_acc, pf, ones, c);
    softmax_probs_slab<M, 1, NQ16>(s_acc, m_run, l_acc, pf, ones, c);

    // O^T += V^T P^T ; lane reads V^T[16*dt + li][keys of slab s, group lg]
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      if (RAGGED && 16 * dt >= d_real) continue;
      const int d = 16 * dt + li;
      const int swz = ((d >> 1) & 7) ^ ((d >> 4) & 7);
#pragma unroll
      for (int s = 0; s < NS; ++s) {
        const vec16 vf = load16(lds_v + d * VPITCH + (((4 * s + lg) ^ swz) << 4));
#pragma unroll
        for (int qt = 0; qt < NQ16; ++qt)
          o_acc[qt][dt] = M::run(vf, pf[qt][s], o_acc[qt][dt]);
      }
    }
    }
    __syncthreads();  // every wave is done with this tile before it is overwritten
  }

  // ---- epilogue: normalise and store O[query li][16*dt + 4*lg .. +4] ------------
#pragma unroll
  for (int qt = 0; qt < NQ16; ++qt) {
    if (qt < nq_valid) {
      const float l = l_acc[qt][0];
      const float inv = l > 0.0f ? 1.0f / l : 1.0f;
      const int qr = q_wave0 + qt * 16 + li;
      if (qr < q_len) {
        char *dst = out_base + (int64_t)qr * p.o_token_bytes + 4 * lg * 2;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
          if (RAGGED && 16 * dt >= d_real) continue;
          uint2 val;
          val.x = M::pack2(o_acc[qt][dt][0] * inv, o_acc[qt][dt][1] * inv);
          val.y = M::pack2(o_acc[qt][dt][2] * inv, o_acc[qt][dt][3] * inv);
          *reinterpret_cast<uint2 *>(dst + 16 * dt * 2) = val;
        }
      }
    }
  }
}


// ---------------------------------------------------------------------------
// DMA variant (plain and query-side modes): K/V rows go global -> LDS directly
// (global_load_lds, 16 B per lane, no staging registers) into a two-deep ring,
// and V^T fragments are produced by the LDS transpose read ds_read_b64_tr_b16,
// so V stays row-major and needs no register transpose.
//
// LDS tile layout: [BN rows][D*2 bytes], unpadded; the 16-byte chunk c of row r
// sits at chunk position c ^ f(r).  The permutation is applied on the global
// side (each lane fetches the chunk that belongs at its LDS position), so the
// DMA writes stay linear.  f_K(r) = (r/RW) % CH makes the 16 rows of a K
// fragment read (ds_read_b128) hit 16 different bank groups; f_V(r) =
// 2*((r/RW) % (CH/2)) does the same for the 16 rows x 32 B of a transpose read.
// RW = rows per 256-byte bank window, CH = chunks per row.
//
// ds_read_b64_tr_b16 within a 16-lane group: lane l supplies the address of
// 4 consecutive 16-bit elements; lane i receives element i%4 of the lanes
// 4*j + i/4, j = 0..3.  With lane l pointing at V[row0 + l/4][d0 + 4*(l%4)] lane i
// gets V[row0 + 0..3][d0 + i]: four keys of one column, i.e. half of an MFMA
// A-operand of V^T.
// One query tile of one (request, head): the NW waves (4 in every instantiation; the tile geometry below is
// written in terms of NW so that it stays in one place) take WQ = 16 * NQ16 query rows each, starting at row
// q_tile0 of the request, and stream the request's key tiles [t_begin, t_end) through the LDS ring.
template <int DTYPE, int D, int NQ16, int MODE, int NW = 4, bool SMALL = false, int KSPLIT = 1>
__device__ __forceinline__ void attn_dma_part(const AttnParams &p, char *lds_k0, char *lds_v0, char *lds_k1,
                                              char *lds_v1, float *lds_rope, int b, int q_begin, int q_len, int q_tile0,
                                              int head, int kvh, int kv_begin, int kv_len, int t_begin, int t_end) {
  constexpr int BN = 64;
  constexpr int WQ = 16 * NQ16;
  constexpr int KS = D / 32;
  constexpr int NT = BN / 16;
  constexpr int DT = D / 16;
  constexpr int NS = BN / 32;
  constexpr int ROW_BYTES = D * 2;
  constexpr int CH = ROW_BYTES / 16;          // chunks per row: 16 (D=128) or 8 (D=64)
  constexpr int RW = 256 / ROW_BYTES;         // rows per bank window: 1 or 2
  constexpr int RPI = 64 / CH;                // rows per DMA instruction: 4 or 8
  constexpr int WAVE_ROWS = BN / NW;          // rows of every tile that each of the NW waves copies (16 or 8)
  constexpr int THREADS = 64 * NW;
  constexpr int NI = WAVE_ROWS / RPI;         // DMA instructions per wave, tile and tensor: 4 or 2
  constexpr int TILE_BYTES = BN * ROW_BYTES;
  // KSPLIT = 2 (query tiles of at most half the rows): waves 2g and 2g + 1 hold the same WQ query rows and take
  // the first and the second 32 keys of every tile; their partial (reference, denominator, O) triples are merged
  // through LDS behind the key loop.  Every wave still copies its 16 rows of each tile.
  static_assert(KSPLIT == 1 || (KSPLIT == 2 && NW == 4), "key split: one or two waves per query row group");
  // Short query tiles have too little work per key tile to hide a copy issued in the middle of it: all copies of
  // the next tile go out right behind the barrier.
  constexpr bool COPY_EARLY = KSPLIT == 2;
  constexpr int NTL = NT / KSPLIT;            // 16-key blocks of a tile that a wave scores
  constexpr int NSL = NS / KSPLIT;            // 32-key slabs of a tile that a wave multiplies into O
  using M = Mma<DTYPE>;
  typedef short s16x4 __attribute__((ext_vector_type(4)));
  // An opaque zero keeps the compiler from computing the lane-derived address constants below ahead of the
  // kernel's set-up code (the tile lookup), where they would only lengthen live ranges: one scalar move, and
  // measured 3 % on the relocation modes (query-side 115 vs 118 µs on the relocated anchor-recompute shape).
  int opaque_zero;
  asm volatile("s_mov_b32 %0, 0" : "=s"(opaque_zero));
  const int tid = threadIdx.x + opaque_zero;
  const int lane = tid & 63, wave = tid >> 6;
  const int li = lane & 15, lg = lane >> 4;
  const int kp = KSPLIT == 1 ? 0 : __builtin_amdgcn_readfirstlane(wave % KSPLIT);  // which part of a tile's keys
  const int q_wave0 = q_tile0 + (wave / KSPLIT) * WQ;
  int nq_valid = (q_len - q_wave0 + 15) / 16;
  nq_valid = nq_valid < 0 ? 0 : (nq_valid > NQ16 ? NQ16 : nq_valid);
  char *out_base = p.out + (int64_t)q_begin * p.o_token_bytes + (int64_t)head * p.o_head_bytes;

  if (kv_len <= 0) {
    for (int r = tid / CH; r < NW / KSPLIT * WQ; r += THREADS / CH) {
      const int qr = q_tile0 + r;
      if (qr < q_len) store16(out_base + (int64_t)qr * p.o_token_bytes + (tid % CH) * 16, vec16{{0, 0, 0, 0}});
    }
    return;
  }

  int shared_len = 0, shift = 0;
  if (MODE == MODE_QUERY_SIDE) {
    shared_len = p.shared_kv_lens[b];
    shared_len = shared_len < 0 ? 0 : (shared_len > kv_len ? kv_len : shared_len);
    shift = p.affix_shifts[b];
    if (shift < 0 || shift >= p.rope_rows) shift = 0;
  }

  const int tiles_a = (shared_len + BN - 1) / BN;

  // Query fragments (B operand).  Query-side mode scores the shared keys, which come first,
  // against the rotated query q' and everything after them against q itself; only one of the
  // two is live at a time: q' is built here and q is re-read when the shared tiles are done.
  vec16 qf[NQ16][KS];
  const char *q_base = p.q + (int64_t)q_begin * p.q_token_bytes + (int64_t)head * p.q_head_bytes;
  auto load_q = [&](bool rotated) __attribute__((always_inline)) {
#pragma unroll
    for (int qt = 0; qt < NQ16; ++qt) {
      const int qr = q_wave0 + qt * 16 + li;
      const bool live = qr < q_len;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
        qf[qt][ks] = live ? load16(q_base + (int64_t)qr * p.q_token_bytes + (32 * ks + 8 * lg) * 2)
                          : vec16{{0, 0, 0, 0}};
      if (MODE == MODE_QUERY_SIDE && rotated && shift != 0) {
        const float *cr = p.cos_tab + (int64_t)shift * D;
        const float *sr = p.sin_tab + (int64_t)shift * D;
#pragma unroll
        for (int ks = 0; ks < KS / 2; ++ks)
          rotate_pair<DTYPE, D>(qf[qt][ks], qf[qt][ks + KS / 2], cr, sr, 32 * ks + 8 * lg, -1.0f);
      }
    }
  };
  load_q(MODE == MODE_QUERY_SIDE && t_begin < tiles_a);

  // ---- DMA bookkeeping: this lane's row and chunk inside each of its NI instructions
  const int dma_row0 = wave * WAVE_ROWS + lane / CH;   // + i*RPI
  const int dma_chunk = lane % CH;
  // wave-uniform, and said so: the copies take them as scalar operands
  const char *kc_base = uniform_ptr(p.k_cache + (int64_t)kvh * p.kv_head_bytes);
  const char *vc_base = uniform_ptr(p.v_cache + (int64_t)kvh * p.kv_head_bytes);

  // slots of this lane's rows: even tiles in slot_a, odd tiles in slot_b (two named
  // register arrays, indexed statically).  load_slots only issues the loads; the
  // values are first touched by issue() one barrier later, so no wait for them is
  // ever placed in front of the MFMA work.
  int slot_a[NI], slot_b[NI];
  const int32_t *const slot_lane = p.slot_map + kv_begin + dma_row0;   // + first key of the tile + i * RPI
  auto load_slots = [&](int t, int (&dst)[NI]) __attribute__((always_inline)) {
    const TileRange tr = tile_range_of(t < t_end ? t : t_end - 1, tiles_a, shared_len, kv_len, BN);
    if (t < t_end && tr.n0 + BN <= tr.n_end) {
      // full tile (a wave-uniform test): one address per lane, the row groups are immediate offsets
      const int32_t *src = slot_lane + tr.n0;
#pragma unroll
      for (int i = 0; i < NI; ++i) dst[i] = src[i * RPI];
    } else {
#pragma unroll
      for (int i = 0; i < NI; ++i) {
        const int n = tr.n0 + dma_row0 + i * RPI;
        // rows past the end of the range read index 0 (kv_len > 0, always readable);
        // issue() ignores the value
        dst[i] = p.slot_map[kv_begin + ((t < t_end && n < tr.n_end) ? n : 0)];
      }
    }
  };
  // Byte offset of this lane's (swizzled) chunk inside row i of a tile; the slot term is added per copy.  SMALL:
  // the cache spans less than 4 GiB and slot numbers and the slot pitch fit 24 bits, so a copy's source is a
  // wave-uniform base plus one 24-bit multiply-add (the 64-bit multiply-add of the general form runs at a
  // quarter of that rate).
  uint32_t k_lane_off[NI], v_lane_off_dma[NI];
#pragma unroll
  for (int i = 0; i < NI; ++i) {
    const int r = dma_row0 + i * RPI;
    k_lane_off[i] = (uint32_t)((dma_chunk ^ ((r / RW) % CH)) << 4);
    v_lane_off_dma[i] = (uint32_t)((dma_chunk ^ (2 * ((r / RW) % (CH / 2)))) << 4);
  }
  const uint32_t slot_pitch = (uint32_t)p.kv_slot_bytes;
  const uint32_t slot_limit = p.num_slots > 0x7fffffffLL ? 0x7fffffffu : (uint32_t)p.num_slots;
  // A tile whose 64 rows all exist and whose slots all lie inside the cache (the common case) is
  // copied row group by row group with issue_rows(), which the compute phase spreads over its
  // own instruction stream: four waves issuing all their copies at once right behind the barrier
  // queue up in the vector memory path for about a thousand cycles, during which they cannot
  // issue anything else.  Every other tile takes issue_slow(): absent rows come from the zero row.
  auto all_present = [&](int t, const int (&slots)[NI]) __attribute__((always_inline)) {
    const TileRange tr = tile_range_of(t, tiles_a, shared_len, kv_len, BN);
    bool in_range = true;  // negative slots wrap to huge unsigned values and fail the range test too
#pragma unroll
    for (int i = 0; i < NI; ++i) in_range &= (uint32_t)slots[i] < slot_limit;
    return tr.n0 + BN <= tr.n_end && __builtin_amdgcn_ballot_w64(!in_range) == 0;
  };
  // this wave's rows inside a tile as a scalar byte offset (the lane's data lands 16 * lane behind the destination)
  const uint32_t wave_dst = __builtin_amdgcn_readfirstlane((uint32_t)(wave * WAVE_ROWS * ROW_BYTES));
  auto issue_rows = [&](int i, char *kbuf, char *vbuf, const int (&slots)[NI]) __attribute__((always_inline)) {
    const uint32_t dst = wave_dst + i * RPI * ROW_BYTES;
    if (SMALL) {
      const uint32_t row_off = __umul24((uint32_t)slots[i], slot_pitch);
      lds_dma16_off(kc_base, row_off + k_lane_off[i], lds_offset_of(kbuf) + dst);
      lds_dma16_off(vc_base, row_off + v_lane_off_dma[i], lds_offset_of(vbuf) + dst);
    } else {
      const uint64_t row_off = (uint64_t)(uint32_t)slots[i] * slot_pitch;
      lds_dma16_at(kc_base + (row_off + k_lane_off[i]), lds_offset_of(kbuf) + dst);
      lds_dma16_at(vc_base + (row_off + v_lane_off_dma[i]), lds_offset_of(vbuf) + dst);
    }
  };
  auto issue_slow = [&](int t, char *kbuf, char *vbuf, const int (&slots)[NI]) __attribute__((always_inline)) {
    const TileRange tr = tile_range_of(t, tiles_a, shared_len, kv_len, BN);
    const char *zero = reinterpret_cast<const char *>(kZeroRow) + (dma_chunk << 4);
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      const int r = dma_row0 + i * RPI;
      const bool present = tr.n0 + r < tr.n_end && (uint32_t)slots[i] < slot_limit;
      const uint64_t row_off = (uint64_t)(uint32_t)slots[i] * slot_pitch;
      const char *ksrc = present ? kc_base + (row_off + k_lane_off[i]) : zero;
      const char *vsrc = present ? vc_base + (row_off + v_lane_off_dma[i]) : zero;
      lds_dma16_at(ksrc, lds_offset_of(kbuf) + wave_dst + i * RPI * ROW_BYTES);
      lds_dma16_at(vsrc, lds_offset_of(vbuf) + wave_dst + i * RPI * ROW_BYTES);
    }
  };
  auto issue = [&](int t, char *kbuf, char *vbuf, const int (&slots)[NI]) __attribute__((always_inline)) {
    if (all_present(t, slots)) {
#pragma unroll
      for (int i = 0; i < NI; ++i) issue_rows(i, kbuf, vbuf, slots);
    } else {
      issue_slow(t, kbuf, vbuf, slots);
    }
  };

  // m_run: reference point of the running sums in log2 units (score * scale * log2 e)
  float m_run[NQ16];
  f32x4 o_acc[NQ16][DT], l_acc[NQ16];
  const float c = p.scale_log2e;
#pragma unroll
  for (int qt = 0; qt < NQ16; ++qt) {
    m_run[qt] = -INFINITY;
    l_acc[qt] = f32x4{0, 0, 0, 0};
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) o_acc[qt][dt] = f32x4{0, 0, 0, 0};
  }
  const uint32_t one2 = M::pack2(1.0f, 1.0f);
  const vec16 ones{{one2, one2, one2, one2}};

  // lane-constant pieces of the fragment addresses
  const int k_swz = (li / RW) % CH;                       // f_K of rows 16*nt + li
  const int v_j = li >> 2, v_ib = li & 3;                 // transpose-read role inside the 16-lane group
  const int v_row = 4 * lg + v_j;                         // + 32*s (+16 for the second half)
  const int v_swz = ((v_row / RW) % (CH / 2));            // f_V(row)/2; rows differ by multiples of 16
  const int v_lane_off = v_row * ROW_BYTES + ((v_ib >> 1) << 4) + ((v_ib & 1) << 3);
  // LDS addresses of this lane's fragments inside the ring's first K tile: the tile (K0, V0, K1, V1 lie 16 KiB
  // apart), the 16-key block and the slab are immediates of the read instructions
  typedef __attribute__((address_space(3))) const char *LdsBytes;
  LdsBytes k_frag[KS], v_frag[DT];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks)
    k_frag[ks] = (LdsBytes)lds_k0 + (li * ROW_BYTES + (((4 * ks + lg) ^ k_swz) << 4) + kp * (BN / KSPLIT) * ROW_BYTES);
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
    v_frag[dt] = (LdsBytes)lds_k0 + (v_lane_off + (((dt ^ v_swz) & (CH / 2 - 1)) << 5) + kp * (BN / KSPLIT) * ROW_BYTES);

  // MASKED = true: keys at tile rows >= n_valid are absent (last tile of a range) and get score -inf.
  // stepped: the copies of the next tile (into nk / nv, slots nslots) ride along, one row group at
  // each of four points of this tile's work.
  auto compute = [&]<bool MASKED>(const char *kbuf, const char *vbuf, int n_valid, bool stepped, char *nk,
                                  char *nv, const int (&nslots)[NI]) __attribute__((always_inline)) {
    auto copy_point = [&](int point) __attribute__((always_inline)) {
      if (stepped) {
#pragma unroll
        for (int i = 0; i < NI; ++i)
          if ((COPY_EARLY ? 0 : i * 4 / NI) == point) issue_rows(i, nk, nv, nslots);
      }
    };
    f32x4 s_acc[NQ16][NTL];
#pragma unroll
    for (int qt = 0; qt < NQ16; ++qt)
#pragma unroll
      for (int nt = 0; nt < NTL; ++nt) s_acc[qt][nt] = f32x4{0, 0, 0, 0};
    auto scores = [&](const vec16 (&qq)[NQ16][KS]) __attribute__((always_inline)) {
#pragma unroll
      for (int nt = 0; nt < NTL; ++nt) {
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
          typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
          const u32x4 kraw = *(__attribute__((address_space(3))) const u32x4 *)(k_frag[ks] + ((kbuf - lds_k0) + 16 * nt * ROW_BYTES));
          const vec16 kf{{kraw.x, kraw.y, kraw.z, kraw.w}};
#pragma unroll
          for (int qt = 0; qt < NQ16; ++qt)
            s_acc[qt][nt] = M::run(kf, qq[qt][ks], s_acc[qt][nt]);
        }
      }
    };
    copy_point(0);
    __builtin_amdgcn_s_setprio(1);
    scores(qf);
    // Issue order of this region: K fragments are read four fragments (eight matrix
    // instructions) ahead of their use, so LDS latency hides behind the matrix core.
    __builtin_amdgcn_sched_group_barrier(0x100, 4, 0);
#pragma unroll
    for (int i = 0; i < (NTL * KS - 4) / 2; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, 2 * NQ16, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
    }
    __builtin_amdgcn_sched_group_barrier(0x008, 4 * NQ16, 0);
    __builtin_amdgcn_s_setprio(0);

    copy_point(1);
    softmax_reference<NQ16, NQ16, NTL, DT, MASKED>(s_acc, m_run, l_acc, o_acc, c, n_valid - kp * (BN / KSPLIT), lg);
    copy_point(2);

    // O^T += V^T P^T, one 32-key slab at a time, so that the exponentials of the second slab
    // have the matrix-core work of the first to hide behind.
    static_assert(NS == 2, "two 32-key slabs per tile");
    vec16 pf[NQ16][NSL];
    auto pv_slab = [&](int s) __attribute__((always_inline)) {
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) {
        const LdsBytes src = v_frag[dt] + ((vbuf - lds_k0) + 32 * s * ROW_BYTES);
        const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3))) *)src);
        const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
            (s16x4 __attribute__((address_space(3))) *)(src + 16 * ROW_BYTES));
        const uint2 lo2 = __builtin_bit_cast(uint2, lo), hi2 = __builtin_bit_cast(uint2, hi);
        const vec16 vf{{lo2.x, lo2.y, hi2.x, hi2.y}};  // the two 64-bit results are the operand as is
#pragma unroll
        for (int qt = 0; qt < NQ16; ++qt)
          o_acc[qt][dt] = M::run(vf, pf[qt][s], o_acc[qt][dt]);
      }
    };
    softmax_probs_slab<M, 0, NQ16>(s_acc, m_run, l_acc, pf, ones, c);
    copy_point(3);
    __builtin_amdgcn_s_setprio(1);
    pv_slab(0);  // with a key split this is the wave's own slab: its offset is part of v_frag
    if constexpr (NSL == 2) {
      softmax_probs_slab<M, 1, NQ16>(s_acc, m_run, l_acc, pf, ones, c);
      pv_slab(1);
    }
    // Issue order: V fragments two d-tiles ahead of their use.
    __builtin_amdgcn_sched_group_barrier(0x100, 4, 0);
#pragma unroll
    for (int i = 0; i < NSL * DT - 2; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, NQ16, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
    }
    __builtin_amdgcn_sched_group_barrier(0x008, (NSL + 1) * NQ16, 0);
    __builtin_amdgcn_s_setprio(0);
  };

  // Key-side relocation: the rows of tile t whose slot lies in the shared range are re-rotated in place, in
  // LDS, right after the tile has landed — once per workgroup and key tile, with the arithmetic of the
  // stand-alone relocation kernel (products and sum rounded separately, one rounding to the cache type), so
  // attention over the rotated tile equals attention over a materialised copy bit for bit.  Thread -> (row
  // tid / 4, a quarter of the row's chunk pairs); chunk c of row r sits at chunk position c ^ f_K(r).
  // Every shared row has its own shift n - slot; in the engine's layouts all shared rows of a request have the
  // shift the caller also passes per request, so the cos / sin rows of that shift are kept in LDS (lds_rope,
  // filled below) and only rows with another shift fetch their own rows from the table.  The row's slot is
  // fetched one tile ahead (rot_slot), behind the compute phase of the tile before.  A thread's row is one of
  // the rows its own wave copied (tid / 4 lies in the wave's 16 rows), so the rotation starts as soon as the
  // wave's own copies have landed and the barrier that publishes the tile publishes the rotated rows.
  constexpr int PAIRS = CH / 2;                    // (d, d + D/2) chunk pairs per row
  constexpr int PER_THREAD = BN * PAIRS / THREADS;  // 2 (D = 128, 4 waves)
  static_assert(BN * PAIRS % THREADS == 0 && PER_THREAD >= 1, "one or more chunk pairs per thread");
  const int rot_row = tid / (PAIRS / PER_THREAD);
  static_assert(64 / (PAIRS / PER_THREAD) == WAVE_ROWS, "a wave rotates exactly the rows it copies");
  int shift0 = 0;
  if (MODE == MODE_KEY_SIDE) {
    shift0 = p.affix_shifts[b];
    if (shift0 < 0 || shift0 >= p.rope_rows) shift0 = 0;
    if (tid < 2 * D / 4) {  // cos row, then sin row: D floats each, 16 bytes per thread
      const float *src = (tid < D / 4 ? p.cos_tab : p.sin_tab) + (int64_t)shift0 * D + (tid % (D / 4)) * 4;
      store16(lds_rope + tid * 4, load16(src));
    }
    __syncthreads();  // the first rotation reads these rows before the first tile's barrier
  }
  auto rot_prefetch = [&](int t) __attribute__((always_inline)) {
    const int n = t * BN + rot_row;
    return MODE == MODE_KEY_SIDE && t < t_end && n < kv_len ? p.slot_map[kv_begin + n] : -1;
  };
  auto rotate_shared_rows = [&](char *kbuf, int t, int slot) __attribute__((always_inline)) {
    const int n = t * BN + rot_row;
    const int delta = n - slot;
    const int ad = delta < 0 ? -delta : delta;
    if (n < kv_len && slot >= 0 && slot < p.shared_prefix_len && delta != 0 && ad < p.rope_rows) {
      char *row = kbuf + rot_row * ROW_BYTES;
      const int f = (rot_row / RW) % CH;
      auto rotate_with = [&](const float *cr, const float *sr, float sign) __attribute__((always_inline)) {
        // a real loop: unrolled, the loads of both chunk pairs are hoisted to the front and the kernel spills
        // (21 registers, 12 % slower in key-side mode)
#pragma nounroll
        for (int k = 0; k < PER_THREAD; ++k) {
          const int c = (tid % (PAIRS / PER_THREAD)) * PER_THREAD + k;
          char *lo_p = row + ((c ^ f) << 4), *hi_p = row + (((c + PAIRS) ^ f) << 4);
          vec16 lo = load16(lo_p), hi = load16(hi_p);
          rotate_pair_half_fast<DTYPE>(lo, hi, cr, sr, c * 8, D / 2, sign);
          store16(lo_p, lo);
          store16(hi_p, hi);
        }
      };
      // separate calls: LDS reads here, global loads there.  The cached rows belong to shift0 >= 0, so their sign
      // is the literal +1 and the multiplications by it fold away.
      if (delta == shift0) rotate_with(lds_rope, lds_rope + D, 1.0f);
      else rotate_with(p.cos_tab + (int64_t)ad * D, p.sin_tab + (int64_t)ad * D, delta < 0 ? -1.0f : 1.0f);
    }
  };
  int rot_slot = rot_prefetch(t_begin);

  // ---- two-deep ring: tile t lives in buffer (t - t_begin) & 1 -----------------------
  // Full tiles run in the loop without any masking code.  In plain mode the one partial tile (the
  // tail of the key range) is peeled off behind the loop; with query-side relocation the shared
  // range may end in a partial tile in the middle, so every tile takes the masked form there.
  constexpr bool PEEL_TAIL = MODE != MODE_QUERY_SIDE;
  const int n_full = kv_len / BN;
  const int t_stop = PEEL_TAIL ? (t_end < n_full ? t_end : n_full) : t_end;  // tiles handled inside the loop
  load_slots(t_begin, slot_a);
  issue(t_begin, lds_k0, lds_v0, slot_a);
  load_slots(t_begin + 1, slot_b);
  for (int t = t_begin; t < t_stop; t += 2) {
    // first tile of the pair: wait for its copies, publish it, start the second, compute
    __builtin_amdgcn_s_waitcnt(0);  // this wave's copies of tile t have landed
    if (MODE == MODE_KEY_SIDE) {
      const int cur = rot_slot;
      rot_slot = rot_prefetch(t + 1);
      rotate_shared_rows(lds_k0, t, cur);
    }
    __syncthreads();                // ... and everybody else's; buffer 1 is no longer being read
    bool stepped = false;
    if (t + 1 < t_end) {
      load_slots(t + 2, slot_a);    // slot loads go first: vmcnt retires in order, so waiting
      stepped = all_present(t + 1, slot_b);  // for them later never waits for the copies behind them
      if (!stepped) issue_slow(t + 1, lds_k1, lds_v1, slot_b);
    }
    if (nq_valid > 0) {
      if (MODE == MODE_QUERY_SIDE && t == tiles_a && t > t_begin) load_q(false);  // shared keys done: back to q
      const TileRange tr = tile_range_of(t, tiles_a, shared_len, kv_len, BN);
      compute.template operator()<!PEEL_TAIL>(lds_k0, lds_v0, tr.n_end - tr.n0, stepped, lds_k1, lds_v1, slot_b);
    } else if (stepped) {
#pragma unroll
      for (int i = 0; i < NI; ++i) issue_rows(i, lds_k1, lds_v1, slot_b);
    }
    if (t + 1 >= t_stop) break;
    __builtin_amdgcn_s_waitcnt(0);
    if (MODE == MODE_KEY_SIDE) {
      const int cur = rot_slot;
      rot_slot = rot_prefetch(t + 2);
      rotate_shared_rows(lds_k1, t + 1, cur);
    }
    __syncthreads();
    stepped = false;
    if (t + 2 < t_end) {
      load_slots(t + 3, slot_b);
      stepped = all_present(t + 2, slot_a);
      if (!stepped) issue_slow(t + 2, lds_k0, lds_v0, slot_a);
    }
    if (nq_valid > 0) {
      if (MODE == MODE_QUERY_SIDE && t + 1 == tiles_a) load_q(false);
      const TileRange tr = tile_range_of(t + 1, tiles_a, shared_len, kv_len, BN);
      compute.template operator()<!PEEL_TAIL>(lds_k1, lds_v1, tr.n_end - tr.n0, stepped, lds_k0, lds_v0, slot_a);
    } else if (stepped) {
#pragma unroll
      for (int i = 0; i < NI; ++i) issue_rows(i, lds_k0, lds_v0, slot_a);
    }
  }
  if (PEEL_TAIL && t_stop < t_end) {  // tail tile t_stop: its copies were issued one step earlier
    __builtin_amdgcn_s_waitcnt(0);
    const bool odd = ((t_stop - t_begin) & 1) != 0;
    if (MODE == MODE_KEY_SIDE) rotate_shared_rows(odd ? lds_k1 : lds_k0, t_stop, rot_slot);
    __syncthreads();
    if (nq_valid > 0)
      compute.template operator()<true>(odd ? lds_k1 : lds_k0, odd ? lds_v1 : lds_v0, kv_len - t_stop * BN, false,
                                        nullptr, nullptr, slot_a);
  }
  __syncthreads();  // every wave is done reading the K/V ring

  // ---- key split: the odd wave of a pair hands its partial state to the even one ---------------
  // Both waves hold the same queries in the same lanes, so the merge is lane-local.  The odd wave parks O (fp32,
  // in register order: exactly one ring buffer) in its own output-staging buffer and (reference, denominator)
  // at the end of its partner's; a wave that never saw a key (requests of at most 32 keys) reports -inf.
  if constexpr (KSPLIT == 2) {
    static_assert(NQ16 * DT * 64 * 16 <= TILE_BYTES, "a wave's partial O must fit one ring buffer");
    f32x4 *xo = reinterpret_cast<f32x4 *>(lds_k0 + (wave | 1) * TILE_BYTES);
    // (the last KiB of the even wave's buffer: its output staging below uses less than the first 9 KiB)
    static_assert(WQ * (ROW_BYTES + 16) + NQ16 * 2 * 64 * 4 <= TILE_BYTES, "room for the exchanged statistics");
    float *xml = reinterpret_cast<float *>(lds_k0 + ((wave & ~1) + 1) * TILE_BYTES - NQ16 * 2 * 64 * 4);
    if (kp == 1) {
#pragma unroll
      for (int qt = 0; qt < NQ16; ++qt) {
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) xo[(qt * DT + dt) * 64 + lane] = o_acc[qt][dt];
        xml[(2 * qt) * 64 + lane] = kv_len > BN / KSPLIT ? m_run[qt] : -INFINITY;
        xml[(2 * qt + 1) * 64 + lane] = l_acc[qt][0];
      }
    }
    __syncthreads();
    if (kp == 1) return;
#pragma unroll
    for (int qt = 0; qt < NQ16; ++qt) {
      const float m1 = xml[(2 * qt) * 64 + lane], l1 = xml[(2 * qt + 1) * 64 + lane];
      const float ms = fmaxf(m_run[qt], m1);
      const float a0 = __builtin_amdgcn_exp2f(m_run[qt] - ms), a1 = __builtin_amdgcn_exp2f(m1 - ms);
      l_acc[qt][0] = l_acc[qt][0] * a0 + l1 * a1;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) o_acc[qt][dt] = o_acc[qt][dt] * a0 + xo[(qt * DT + dt) * 64 + lane] * a1;
    }
  }

  // ---- epilogue: normalise, transpose through LDS, store whole 16-byte chunks ------------------
  // Lane layout of O^T (query li, features 16*dt + 4*lg .. +4) would give 8-byte stores scattered
  // over 16 rows; staging the wave's WQ x D tile in LDS (one 16 KiB ring buffer per wave, rows padded
  // to 272 B against bank conflicts) lets 16 consecutive lanes write one full output row.
  {
    constexpr int OPITCH = ROW_BYTES + 16;
    // the four ring buffers are one block; the callers make it at least NW * WQ * OPITCH bytes
    static_assert(NW != 4 || WQ * OPITCH <= TILE_BYTES, "per-wave output staging must fit one ring buffer");
    char *stage = lds_k0 + wave * (NW == 4 ? TILE_BYTES : WQ * OPITCH);
#pragma unroll
    for (int qt = 0; qt < NQ16; ++qt) {
      const float l = l_acc[qt][0];
      const float inv = l > 0.0f ? 1.0f / l : 1.0f;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) {
        uint2 val;
        val.x = M::pack2(o_acc[qt][dt][0] * inv, o_acc[qt][dt][1] * inv);
        val.y = M::pack2(o_acc[qt][dt][2] * inv, o_acc[qt][dt][3] * inv);
        *reinterpret_cast<uint2 *>(stage + (qt * 16 + li) * OPITCH + (16 * dt + 4 * lg) * 2) = val;
      }
    }
    // same wave wrote and reads: LDS accesses of one wave are ordered, no barrier needed
    constexpr int ROWS_PER_PASS = 64 / CH;
#pragma unroll
    for (int r0 = 0; r0 < WQ; r0 += ROWS_PER_PASS) {
      const int r = r0 + lane / CH;
      const int qr = q_wave0 + r;
      if (qr < q_len) {
        const vec16 v = load16(stage + r * OPITCH + (lane % CH) * 16);
        store16(out_base + (int64_t)qr * p.o_token_bytes + (lane % CH) * 16, v);
      }
    }
  }
}

// Key tiles of request b as attn_dma_part walks them (query-side mode: the shared range and the rest are tiled
// separately); a request without keys keeps one virtual tile so that somebody owns its (zero) output rows.
template <int MODE>
__device__ __forceinline__ int sk_key_tiles(const AttnParams &p, int b, int kv_len) {
  if (kv_len <= 0) return 1;
  if (MODE != MODE_QUERY_SIDE) return (kv_len + 63) / 64;
  int shared = p.shared_kv_lens[b];
  shared = shared < 0 ? 0 : (shared > kv_len ? kv_len : shared);
  return (shared + 63) / 64 + (kv_len - shared + 63) / 64;
}

// One workgroup per unit, units dealt whole: blocks are handed out in index order, which with the
// longest-request-first tile order of locate_query_tile_lpt is longest-processing-time-first list scheduling.
template <int DTYPE, int D, int MODE, bool SMALL, int NW = 4>
__global__ __launch_bounds__(64 * NW, NW == 4 ? 2 : 1) void varlen_attn_unit_kernel(AttnParams p) {
  constexpr int BM = 32 * NW;
  constexpr int TILE_BYTES = 64 * D * 2;
  constexpr int STAGING = NW * 32 * (D * 2 + 16);
  // one block, so that the ring keeps its 1 KiB alignment (the swizzle that makes the fragment reads
  // conflict-free counts on it)
  // (+ the cos / sin rows of the request's shift in key-side mode)
  __shared__ __attribute__((aligned(1024))) char lds[(4 * TILE_BYTES > STAGING ? 4 * TILE_BYTES : STAGING) +
                                                     (MODE == MODE_KEY_SIDE ? 2 * D * 4 : 0)];
  float *const lds_rope = reinterpret_cast<float *>(lds + (4 * TILE_BYTES > STAGING ? 4 * TILE_BYTES : STAGING));
  char *const lds_k0 = lds, *const lds_v0 = lds + TILE_BYTES;
  char *const lds_k1 = lds + 2 * TILE_BYTES, *const lds_v1 = lds + 3 * TILE_BYTES;
  int tile, kvh, hg;
  const int group = p.H / p.H_kv;
  int b = 0, q_begin = 0, q_len = 0, kv_begin = 0, kv_len = 0;
  if (p.plan) {
    // The caller's dispatch plan names this block's unit.  Every field is checked against the call's own
    // sizes, so a plan made for other lengths can leave rows unwritten but cannot send an access astray.
    const int2 e = reinterpret_cast<const int2 *>(p.plan)[blockIdx.x];
    b = __builtin_amdgcn_readfirstlane(e.x);
    const unsigned th = (unsigned)__builtin_amdgcn_readfirstlane(e.y);
    if ((unsigned)b >= (unsigned)p.B) return;
    tile = (int)(th & 0xfffffu);
    const int planned_head = (int)(th >> 20);
    if (planned_head >= p.H) return;
    kvh = planned_head / group;
    hg = planned_head - kvh * group;
    q_begin = p.cu_q[b];
    q_len = p.cu_q[b + 1] - q_begin;
    kv_begin = p.cu_k[b];
    kv_len = p.cu_k[b + 1] - kv_begin;
    if (tile * BM >= q_len) return;
  } else {
    if (!block_to_tile_head(p, tile, kvh, hg)) return;
    int tile_in_request = 0;
    if (p.B <= 64) {
      if (!locate_query_tile_lpt(p.cu_q, p.cu_k, p.B, BM, tile, b, q_begin, q_len, tile_in_request, kv_begin, kv_len)) return;
    } else {
      if (!locate_query_tile(p.cu_q, p.B, BM, tile, b, q_begin, q_len, tile_in_request)) return;
      kv_begin = p.cu_k[b];
      kv_len = p.cu_k[b + 1] - kv_begin;
    }
    tile = tile_in_request;
  }
  const int head = kvh * group + hg;
  const int q_tile0 = tile * BM;
  const int kt = sk_key_tiles<MODE>(p, b, kv_len);
  // tiles with at most 64 (32) live rows: two waves per 32 (16) rows, each on half of every tile's keys
  if (q_len - q_tile0 <= BM / 4)
    attn_dma_part<DTYPE, D, 1, MODE, NW, SMALL, 2>(p, lds_k0, lds_v0, lds_k1, lds_v1, lds_rope, b, q_begin, q_len,
                                                   q_tile0, head, kvh, kv_begin, kv_len, 0, kt);
  else if (q_len - q_tile0 <= BM / 2)
    attn_dma_part<DTYPE, D, 2, MODE, NW, SMALL, 2>(p, lds_k0, lds_v0, lds_k1, lds_v1, lds_rope, b, q_begin, q_len,
                                                   q_tile0, head, kvh, kv_begin, kv_len, 0, kt);
  else
    attn_dma_part<DTYPE, D, 2, MODE, NW, SMALL>(p, lds_k0, lds_v0, lds_k1, lds_v1, lds_rope, b, q_begin, q_len,
                                                q_tile0, head, kvh, kv_begin, kv_len, 0, kt);
}

template <int DTYPE, int D, int NQ16>
static int launch_attn(const AttnParams &p0, int mode, int64_t total_q, int64_t plan_blocks, hipStream_t stream) {
  AttnParams p = p0;
  // One 4-wave workgroup per (request, 128-row query tile, head), two workgroups per CU.
  p.num_tiles = (int32_t)((total_q + 127) / 128) + p.B;
  const int64_t blocks = p.plan ? plan_blocks : attn_grid_blocks(p);
  if (blocks > 0x7fffffffLL) return fail(ACACHE_E_SHAPE, "varlen_attn: grid too large");
  // 32-bit copy offsets when the whole cache lies within 4 GiB of a head's base and the factors fit 24 bits
  const bool small = p.num_slots < (1 << 24) && p.kv_slot_bytes > 0 && p.kv_slot_bytes < (1 << 24) &&
                     p.num_slots * p.kv_slot_bytes + 4096 <= 0xffffffffLL;
  const dim3 grid((unsigned)blocks), block(256);
#define ACACHE_UNIT(M)                                                                              \
  if (mode == M) {                                                                                  \
    if (small) hipLaunchKernelGGL((varlen_attn_unit_kernel<DTYPE, D, M, true>), grid, block, 0, stream, p); \
    else hipLaunchKernelGGL((varlen_attn_unit_kernel<DTYPE, D, M, false>), grid, block, 0, stream, p);      \
  }
  ACACHE_UNIT(MODE_PLAIN)
  ACACHE_UNIT(MODE_KEY_SIDE)
#undef ACACHE_UNIT
  // query-side mode keeps the 64-bit form: with the scalar bases its kernel runs out of scalar registers and
  // measures 10 % slower
  if (mode == MODE_QUERY_SIDE)
    hipLaunchKernelGGL((varlen_attn_unit_kernel<DTYPE, D, MODE_QUERY_SIDE, false>), grid, block, 0, stream, p);
  return launch_status("varlen_attn_unit_kernel");
}

// Any other head_dim (a multiple of 16 up to 256): the register-staged kernel at a padded width of 256,
// 16 query rows per wave, all three relocation modes.  A correctness path for model shapes outside the two
// tuned widths, not a tuned one.
template <int DTYPE>
static int launch_attn_any_head_dim(const AttnParams &p0, int mode, int64_t total_q, hipStream_t stream) {
  AttnParams p = p0;
  constexpr int BM = 64, DPAD = 256;
  p.num_tiles = (int32_t)((total_q + BM - 1) / BM) + p.B;
  int64_t blocks = (int64_t)p.num_tiles * p.H;
  blocks = (blocks + 7) / 8 * 8;
  if (blocks > 0x7fffffffLL) return fail(ACACHE_E_SHAPE, "varlen_attn: grid too large");
  dim3 grid((unsigned)blocks), block(256);
  switch (mode) {
    case MODE_PLAIN:
      hipLaunchKernelGGL((varlen_attn_kernel<DTYPE, DPAD, 1, MODE_PLAIN, true>), grid, block, 0, stream, p);
      break;
    case MODE_KEY_SIDE:
      hipLaunchKernelGGL((varlen_attn_kernel<DTYPE, DPAD, 1, MODE_KEY_SIDE, true>), grid, block, 0, stream, p);
      break;
    default:
      hipLaunchKernelGGL((varlen_attn_kernel<DTYPE, DPAD, 1, MODE_QUERY_SIDE, true>), grid, block, 0, stream, p);
      break;
  }
  return launch_status("varlen_attn_kernel (any head_dim)");
}

}  // namespace acache

using namespace acache;

extern "C" int acache_varlen_attn_planned(
    void *out, const void *q, const void *k_cache, const void *v_cache, const int32_t *cu_q,
    const int32_t *cu_k, const int32_t *slot_map, float scale, int32_t shared_prefix_len,
    const int32_t *shared_kv_lens, const int32_t *affix_shifts, const float *rope_cos,
    const float *rope_sin, int32_t rope_rows, int32_t B, int64_t total_q, int64_t total_k, int32_t H,
    int32_t H_kv, int32_t D, int32_t dtype, int64_t num_slots, int64_t q_token_stride,
    int64_t q_head_stride, int64_t out_token_stride, int64_t out_head_stride, int64_t kv_slot_stride,
    int64_t kv_head_stride, const int32_t *plan, int64_t plan_blocks, void *stream) {
  if (plan && (plan_blocks <= 0 || ((uintptr_t)plan & 7)))
    return fail(ACACHE_E_SHAPE, "varlen_attn: a plan needs a positive block count and 8-byte alignment");
  if (dtype != ACACHE_BF16 && dtype != ACACHE_F16)
    return fail(ACACHE_E_DTYPE, "varlen_attn: dtype %d not supported (bf16 or f16)", dtype);
  if (D < 16 || D > 256 || D % 16 != 0)
    return fail(ACACHE_E_SHAPE, "varlen_attn: head_dim %d not supported (a multiple of 16 up to 256)", D);
  if (B < 0 || total_q < 0 || total_k < 0 || H <= 0 || H_kv <= 0 || H % H_kv != 0 || num_slots < 0)
    return fail(ACACHE_E_SHAPE, "varlen_attn: bad sizes (H=%d, H_kv=%d)", H, H_kv);
  if (!(scale > 0.0f) || scale > 3.0e38f)
    return fail(ACACHE_E_RANGE, "varlen_attn: softmax scale must be positive and finite");
  if (B == 0 || total_q == 0) return 0;
  if (!out || !q || !cu_q || !cu_k) return fail(ACACHE_E_NULL, "varlen_attn: NULL pointer");
  if (total_k > 0 && (!k_cache || !v_cache || !slot_map))
    return fail(ACACHE_E_NULL, "varlen_attn: NULL cache or slot map");
  const bool relocate = shared_prefix_len > 0 && affix_shifts != nullptr;
  const bool query_side = relocate && shared_kv_lens != nullptr;
  if (relocate && (!rope_cos || !rope_sin || rope_rows <= 0))
    return fail(ACACHE_E_MODE, "varlen_attn: relocation requested without RoPE tables");
  const int es = 2;
  if (!aligned16(out) || !aligned16(q) || !aligned16(k_cache) || !aligned16(v_cache) ||
      (q_token_stride * es) % 16 || (q_head_stride * es) % 16 || (out_token_stride * es) % 16 ||
      (out_head_stride * es) % 16 || (kv_slot_stride * es) % 16 || (kv_head_stride * es) % 16)
    return fail(ACACHE_E_ALIGN, "varlen_attn: pointers and strides must be 16-byte aligned");
  AttnParams p;
  p.out = (char *)out; p.q = (const char *)q;
  p.k_cache = (const char *)k_cache; p.v_cache = (const char *)v_cache;
  p.cu_q = cu_q; p.cu_k = cu_k; p.slot_map = slot_map;
  p.shared_kv_lens = shared_kv_lens; p.affix_shifts = affix_shifts;
  p.cos_tab = rope_cos; p.sin_tab = rope_sin;
  p.plan = (D == 128 || D == 64) ? plan : nullptr;  // the padded-width kernel keeps its own order
  p.scale_log2e = scale * 1.4426950408889634f;
  p.shared_prefix_len = relocate ? shared_prefix_len : 0;
  p.rope_rows = rope_rows; p.B = B; p.H = H; p.H_kv = H_kv; p.num_tiles = 0; p.head_dim = D;
  p.num_slots = num_slots;
  p.q_token_bytes = q_token_stride * es; p.q_head_bytes = q_head_stride * es;
  p.o_token_bytes = out_token_stride * es; p.o_head_bytes = out_head_stride * es;
  p.kv_slot_bytes = kv_slot_stride * es; p.kv_head_bytes = kv_head_stride * es;
  const int mode = query_side ? MODE_QUERY_SIDE : (relocate ? MODE_KEY_SIDE : MODE_PLAIN);
  hipStream_t st = (hipStream_t)stream;
#define ACACHE_ATTN(DT, DD) \
  if (dtype == DT && D == DD) return launch_attn<DT, DD, 2>(p, mode, total_q, plan_blocks, st);
  ACACHE_ATTN(ACACHE_BF16, 128)
  ACACHE_ATTN(ACACHE_BF16, 64)
  ACACHE_ATTN(ACACHE_F16, 128)
  ACACHE_ATTN(ACACHE_F16, 64)
#undef ACACHE_ATTN
  if (dtype == ACACHE_BF16) return launch_attn_any_head_dim<ACACHE_BF16>(p, mode, total_q, st);
  return launch_attn_any_head_dim<ACACHE_F16>(p, mode, total_q, st);
}

extern "C" int acache_varlen_attn(
    void *out, const void *q, const void *k_cache, const void *v_cache, const int32_t *cu_q,
    const int32_t *cu_k, const int32_t *slot_map, float scale, int32_t shared_prefix_len,
    const int32_t *shared_kv_lens, const int32_t *affix_shifts, const float *rope_cos,
    const float *rope_sin, int32_t rope_rows, int32_t B, int64_t total_q, int64_t total_k, int32_t H,
    int32_t H_kv, int32_t D, int32_t dtype, int64_t num_slots, int64_t q_token_stride,
    int64_t q_head_stride, int64_t out_token_stride, int64_t out_head_stride, int64_t kv_slot_stride,
    int64_t kv_head_stride, void *stream) {
  return acache_varlen_attn_planned(out, q, k_cache, v_cache, cu_q, cu_k, slot_map, scale, shared_prefix_len,
                                    shared_kv_lens, affix_shifts, rope_cos, rope_sin, rope_rows, B, total_q, total_k,
                                    H, H_kv, D, dtype, num_slots, q_token_stride, q_head_stride, out_token_stride,
                                    out_head_stride, kv_slot_stride, kv_head_stride, nullptr, 0, stream);
}
