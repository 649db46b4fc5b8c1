// Bidirectional varlen attention for requests with more than 128 query rows (gfx950): wide workgroups on a
// persistent grid.
//
// Workgroup = 8 waves = one per CU.  It owns up to 256 query rows of one (request, head) and streams the
// request's keys in tiles of 64 through a four-deep LDS ring shared by the 8 waves, so the sibling query
// tiles of a head read one copy of K/V instead of two, and every wave issues half the global -> LDS copies
// per matrix instruction that a 4-wave workgroup does.  The 16-row query tiles of the unit are dealt round-robin
// to the waves (wave w takes tiles w and w + 8), so the four SIMDs carry the same load to within one
// tile and a unit of 150 rows costs three quarters of a full one.  Copies run three key tiles ahead of the
// matrix work; the slots of the keys come from an LDS table filled once per stretch of 64 tiles, so the only
// vector-memory instructions in the loop are the copies and the waits can be counted exactly.
//
// Same MFMA formulation, softmax steps and rounding as the 4-wave kernels (attn_common.h): per query row the
// arithmetic does not depend on which kernel or wave handled it.
//
// Schedule.  The grid is one workgroup per CU, not one per unit: the units differ in length by the requests'
// key counts and query-row counts, and dealt out whole they leave a third of the chip idle while the long
// ones finish.  Instead all units of a group of KV heads are laid end to end on one timeline, measured in
// weighted key-tile steps, and every workgroup takes an equal stretch of it, cut at key-tile boundaries: at
// most its first and its last unit are shared with a neighbour.  Since a unit reads its K/V exactly once
// wherever it is cut, cutting costs no extra traffic.  The parts of a cut unit meet in the caller's
// workspace: every part leaves its un-normalised accumulators there and bumps the unit's counter; the part
// that finds all the others already there merges them in part order (a fixed order, so results are bit-stable
// from run to run), resets the counter and writes the output.  Nobody waits for anybody.
#include "attn_common.h"

namespace acache {

constexpr int kWideWaves = 8;
constexpr int kWideThreads = 64 * kWideWaves;
constexpr int kWideRows = 32 * kWideWaves;       // query rows per unit
constexpr int kWideStages = 4;                   // ring depth
constexpr int kWideAhead = kWideStages - 1;      // copies run this many key tiles ahead of the matrix work
constexpr int kWideTableTiles = 64;              // key tiles whose slots the LDS table holds at a time
// partial state of one part: 16 accumulator quads + (m, l) of the two query tiles, per thread, thread-major
constexpr int kWideAccBytes = kWideThreads * 16 * 16;
constexpr int kWideSlotBytes = kWideAccBytes + kWideThreads * 4 * 4;
constexpr int kWideCounterAlign = 4096;

// ---- the timeline ------------------------------------------------------------------------------------------
// Weights in twentieths of a full key-tile step.  A unit weighs kUnit + tiles * c, c by the busiest SIMD's
// share of 16-row query tiles (1 .. 4): matrix and softmax work scale with it, copies and barriers do not.
constexpr int kUnit = 70, kMinStretch = kUnit + 4 * 20;
__device__ __forceinline__ int wide_tile_cost(int rows) {
  const int per_simd = (rows + 63) / 64;  // 16-row tiles on the busiest SIMD
  return per_simd >= 4 ? 20 : per_simd == 3 ? 16 : per_simd == 2 ? 12 : 9;
}

struct WideRequest {
  int q_begin, q_len, nt, kt;
  int w_full, w_last;  // weight of a unit of 256 rows / of the request's last query tile
};

// Key tiles of request b as attn_wide_part walks them (query-side mode: the shared range and the rest are tiled
// separately); a request without keys keeps one virtual tile so that somebody owns its (zero) output rows.
template <int MODE>
__device__ __forceinline__ int wide_key_tiles(const AttnParams &p, int b, int kv_len) {
  if (kv_len <= 0) return 1;
  if (MODE != MODE_QUERY_SIDE) return (kv_len + 63) / 64;
  int shared = p.shared_kv_lens[b];
  shared = shared < 0 ? 0 : (shared > kv_len ? kv_len : shared);
  return (shared + 63) / 64 + (kv_len - shared + 63) / 64;
}

template <int MODE>
__device__ __forceinline__ WideRequest wide_request(const AttnParams &p, int b) {
  WideRequest r;
  r.q_begin = p.cu_q[b];
  r.q_len = p.cu_q[b + 1] - r.q_begin;
  r.nt = r.q_len > 0 ? (r.q_len + kWideRows - 1) / kWideRows : 0;
  r.kt = wide_key_tiles<MODE>(p, b, p.cu_k[b + 1] - p.cu_k[b]);
  r.w_full = kUnit + 20 * r.kt;
  r.w_last = kUnit + wide_tile_cost(r.q_len - (r.nt - 1) * kWideRows) * r.kt;
  return r;
}

__device__ __forceinline__ int64_t wide_request_weight(const WideRequest &r) {
  return r.nt > 0 ? (int64_t)(r.nt - 1) * r.w_full + r.w_last : 0;
}

// The schedule is the same in every lane; saying so keeps it in scalar registers.
__device__ __forceinline__ int64_t uniform64(int64_t v) {
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)(uint64_t)v);
  const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)((uint64_t)v >> 32));
  return (int64_t)(((uint64_t)hi << 32) | lo);
}

// LDS is addressed through explicit address-space-3 pointers here: the ring stage is picked at run time, and
// with generic pointers the compiler falls back to flat-address bookkeeping (waits on the vector-memory counter
// in front of every fragment read, which serialises them behind the copies in flight).
typedef __attribute__((address_space(3))) char lds_char;
typedef __attribute__((address_space(3))) int32_t lds_int;
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ vec16 lds_load16(const lds_char *p) {
  const u32x4 v = *reinterpret_cast<const __attribute__((address_space(3))) u32x4 *>(p);
  return vec16{{v.x, v.y, v.z, v.w}};
}
__device__ __forceinline__ void lds_store8(lds_char *p, uint32_t lo, uint32_t hi) {
  *reinterpret_cast<__attribute__((address_space(3))) u32x2 *>(p) = u32x2{lo, hi};
}
// global -> LDS copy of 16 bytes per lane (see lds_dma16): lane l's bytes land at dst + 16*l, dst wave-uniform
__device__ __forceinline__ void lds_copy16(const char *src, lds_char *dst) {
  const uint32_t base = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)dst);
  asm volatile("s_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(src), "{m0}"(base) : "memory");
}

__device__ __forceinline__ void store_f32x4_agent(void *dst, f32x4 v) {
  // written through to memory at agent scope: parts of a unit run on different XCDs, behind different L2s
  uint64_t *d = reinterpret_cast<uint64_t *>(dst);
  const uint2 a{__float_as_uint(v[0]), __float_as_uint(v[1])}, b{__float_as_uint(v[2]), __float_as_uint(v[3])};
  __hip_atomic_store(d, __builtin_bit_cast(uint64_t, a), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __hip_atomic_store(d + 1, __builtin_bit_cast(uint64_t, b), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void store_f32_agent(float *dst, float v) {
  __hip_atomic_store(dst, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// One planned part, as the planner leaves it in LDS (kPlanInts words) ...
enum { kPartB, kPartQTile0, kPartHead, kPartTBegin, kPartTEnd, kPartNParts, kPartIndex, kPartFirstGid, kPartQBegin,
       kPartQLen, kPlanInts = 12 };
// ... and the call's output / workspace pointers, left in LDS once per workgroup
enum { kParOut = 0, kParOutTokenBytes = 2, kParOutHeadBytes = 4, kParSlots = 6, kParCounters = 8, kParInts = 10 };

__device__ __forceinline__ int lds_uniform(const lds_int *p) { return __builtin_amdgcn_readfirstlane(*p); }
__device__ __forceinline__ int64_t lds_uniform64(const lds_int *p) {
  return (int64_t)(((uint64_t)(uint32_t)lds_uniform(p + 1) << 32) | (uint32_t)lds_uniform(p));
}

// Key tiles [t_begin, t_end) of one unit: up to 256 query rows, starting at row q_tile0, of one (request, head).
// nparts == 1: the range is the whole unit.  nparts > 1: see the file comment; this workgroup holds part `part`,
// the workgroup of part 0 has global index first_gid.
//
// What only the end of the part needs (output pointers, part bookkeeping) is read from LDS again there instead
// of being carried through the key loop: kept in scalar registers it pushes the loop over the scalar budget, and
// the instruction scheduler answers excess pressure by giving up the early issue of the fragment reads.
template <int DTYPE, int D, int MODE>
__device__ __forceinline__ void attn_wide_part(const AttnParams &p, lds_char *lds_ring, lds_int *lds_tbl, lds_int *lds_flag,
                                               const lds_int *entry, const lds_int *lds_par) {
  const int b = lds_uniform(entry + kPartB), q_tile0 = lds_uniform(entry + kPartQTile0);
  const int head = lds_uniform(entry + kPartHead), kvh = head / (p.H / p.H_kv);
  const int t_begin = lds_uniform(entry + kPartTBegin), t_end = lds_uniform(entry + kPartTEnd);
  const int q_begin = lds_uniform(entry + kPartQBegin), q_len = lds_uniform(entry + kPartQLen);
  constexpr int BN = 64;
  constexpr int NQ16 = 2;
  constexpr int KS = D / 32;
  constexpr int NT = BN / 16;
  constexpr int DT = D / 16;
  constexpr int NS = BN / 32;
  constexpr int ROW_BYTES = D * 2;
  constexpr int CH = ROW_BYTES / 16;          // chunks per row: 16 (D=128) or 8 (D=64)
  constexpr int RW = 256 / ROW_BYTES;         // rows per bank window: 1 or 2
  constexpr int RPI = 64 / CH;                // rows per copy instruction: 4 or 8
  constexpr int WAVE_ROWS = BN / kWideWaves;  // 8 rows of every tile belong to each wave
  constexpr int NI = WAVE_ROWS / RPI;         // copy instructions per wave, tile and tensor: 2 or 1
  constexpr int COPIES = 2 * NI;              // ... per wave and tile
  constexpr int TILE_BYTES = BN * ROW_BYTES;
  constexpr int STAGE_BYTES = 2 * TILE_BYTES;  // K tile, then V tile
  static_assert(NI >= 1 && kWideAhead == 3, "copy bookkeeping below is written for a lookahead of three tiles");
  using M = Mma<DTYPE>;
  typedef short s16x4 __attribute__((ext_vector_type(4)));
  // An opaque zero ties the lane-derived constants below to this call: otherwise the compiler hoists them out
  // of the persistent loop around it and spills them to keep them alive across units.
  int opaque_zero;
  asm volatile("s_mov_b32 %0, 0" : "=s"(opaque_zero));
  const int tid = threadIdx.x + opaque_zero;
  const int lane = tid & 63, wave = tid >> 6;
  const int li = lane & 15, lg = lane >> 4;
  const int kv_begin = p.cu_k[b];
  const int kv_len = p.cu_k[b + 1] - kv_begin;
  const int rows = q_len - q_tile0 < kWideRows ? q_len - q_tile0 : kWideRows;
  const int n16 = (rows + 15) / 16;
  const int nq_active = (wave < n16 ? 1 : 0) + (wave + kWideWaves < n16 ? 1 : 0);
  // first row of this wave's query tile qt
  auto tile_row0 = [&](int qt) __attribute__((always_inline)) { return q_tile0 + 16 * (wave + kWideWaves * qt); };

  // the previous unit of this workgroup may still be reading the ring (its output staging), the table and the flag
  __syncthreads();

  if (kv_len <= 0) {
    char *out_base = p.out + (int64_t)q_begin * p.o_token_bytes + (int64_t)head * p.o_head_bytes;
    for (int r = tid / CH; r < rows; r += kWideThreads / CH)
      store16(out_base + (int64_t)(q_tile0 + r) * p.o_token_bytes + (tid % CH) * 16, vec16{{0, 0, 0, 0}});
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

  // Query fragments (B operand).  Query-side mode scores the shared keys, which come first, against the rotated
  // query q' and everything after them against q itself; only one of the two is live at a time.
  vec16 qf[NQ16][KS];
  const char *q_base = p.q + (int64_t)q_begin * p.q_token_bytes + (int64_t)head * p.q_head_bytes;
  auto load_q = [&](bool rotated) __attribute__((always_inline)) {
#pragma unroll
    for (int qt = 0; qt < NQ16; ++qt) {
      const int qr = tile_row0(qt) + li;
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
    // Use every fragment register here, so that the compiler waits for these loads now and not at their first
    // use inside the key loop, where its wait (it cannot see the copies in flight) would drain them every tile.
#pragma unroll
    for (int qt = 0; qt < NQ16; ++qt)
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
        asm volatile("" ::"v"(qf[qt][ks].w[0]), "v"(qf[qt][ks].w[1]), "v"(qf[qt][ks].w[2]), "v"(qf[qt][ks].w[3]));
  };
  load_q(MODE == MODE_QUERY_SIDE && t_begin < tiles_a);

  // ---- copy bookkeeping: this lane's row and chunk inside each of its NI instructions -----------------------
  const int dma_row0 = wave * WAVE_ROWS + lane / CH;  // + i * RPI
  const int dma_chunk = lane % CH;
  const char *kc_base = p.k_cache + (int64_t)kvh * p.kv_head_bytes;
  const char *vc_base = p.v_cache + (int64_t)kvh * p.kv_head_bytes;
  // Per-lane source addresses of row group i, minus the slot term: base + swizzled chunk offset (the chunk c of
  // row r sits at chunk position c ^ f(r) of its LDS row; the permutation is applied on the global side).
  const char *k_lane_src[NI], *v_lane_src[NI];
#pragma unroll
  for (int i = 0; i < NI; ++i) {
    const int r = dma_row0 + i * RPI;
    k_lane_src[i] = kc_base + ((dma_chunk ^ ((r / RW) % CH)) << 4);
    v_lane_src[i] = vc_base + ((dma_chunk ^ (2 * ((r / RW) % (CH / 2)))) << 4);
  }
  const uint32_t slot_pitch = (uint32_t)p.kv_slot_bytes;
  const uint32_t slot_limit = p.num_slots > 0x7fffffffLL ? 0x7fffffffu : (uint32_t)p.num_slots;
  const char *zero_src = reinterpret_cast<const char *>(kZeroRow) + (dma_chunk << 4);

  // One of the COPIES copy instructions of a tile: c = 2 * row group + (0: K, 1: V).  `slots` are this lane's
  // entries of the table (-1: the key does not exist or its slot lies outside the cache: copy the zero row).
  auto issue_copy = [&](int c, lds_char *stage, const int (&slots)[NI], bool all_present) __attribute__((always_inline)) {
    const int i = c >> 1;
    const bool v = (c & 1) != 0;
    const uint64_t row_off = (uint64_t)(uint32_t)slots[i] * slot_pitch;
    lds_char *dst = stage + (v ? TILE_BYTES : 0) + (wave * WAVE_ROWS + i * RPI) * ROW_BYTES;  // wave-uniform
    const char *src = (v ? v_lane_src[i] : k_lane_src[i]) + row_off;
    if (!all_present) src = slots[i] >= 0 ? src : zero_src;
    lds_copy16(src, dst);
  };

  float m_run[NQ16];
  f32x4 o_acc[NQ16][DT], l_acc[NQ16];
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
  const float c = p.scale_log2e;

  // One key tile for the first NQA query tiles of the wave.  Keys at tile rows >= n_valid are absent and get
  // score -inf (a wave-uniform branch skips the masking code on full tiles).  stepped: the copies of tile
  // t + 3 (into `next`, slots nslots) ride along, one at each of four points of this tile's work.
  auto compute = [&]<int NQA>(const lds_char *stage, int n_valid, bool stepped, lds_char *next,
                              const int (&nslots)[NI]) __attribute__((always_inline)) {
    const lds_char *kbuf = stage, *vbuf = stage + TILE_BYTES;
    auto copy_point = [&](int point) __attribute__((always_inline)) {
      if (stepped) {
#pragma unroll
        for (int cc = 0; cc < COPIES; ++cc)
          if (cc * 4 / COPIES == point) issue_copy(cc, next, nslots, true);
      }
    };
    f32x4 s_acc[NQ16][NT];
#pragma unroll
    for (int qt = 0; qt < NQA; ++qt)
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) s_acc[qt][nt] = f32x4{0, 0, 0, 0};
    copy_point(0);
    __builtin_amdgcn_s_setprio(1);
    {
      // K fragments (A operand) are read KAHEAD fragments ahead of their use, so LDS latency hides behind the
      // matrix core.  Fragment f = (nt, ks), ks fastest.
      constexpr int KAHEAD = 4;
      auto k_frag = [&](int f) __attribute__((always_inline)) {
        return lds_load16(kbuf + (16 * (f / KS) + li) * ROW_BYTES + (((4 * (f % KS) + lg) ^ k_swz) << 4));
      };
      vec16 kf[KAHEAD];
#pragma unroll
      for (int f = 0; f < KAHEAD; ++f) kf[f] = k_frag(f);
#pragma unroll
      for (int f = 0; f < NT * KS; ++f) {
#pragma unroll
        for (int qt = 0; qt < NQA; ++qt)
          s_acc[qt][f / KS] = M::run(kf[f % KAHEAD], qf[qt][f % KS], s_acc[qt][f / KS]);
        if (f + KAHEAD < NT * KS) kf[f % KAHEAD] = k_frag(f + KAHEAD);
      }
    }
    __builtin_amdgcn_s_setprio(0);

    copy_point(1);
    softmax_reference<NQA, NQ16, NT, DT, true>(s_acc, m_run, l_acc, o_acc, c, n_valid, lg);
    copy_point(2);

    // O^T += V^T P^T, one 32-key slab at a time, so that the exponentials of the second slab have the
    // matrix-core work of the first to hide behind.
    static_assert(NS == 2, "two 32-key slabs per tile");
    vec16 pf[NQ16][NS];
    // V^T fragments (A operand) of d tile dt, keys of slab s: two transpose reads
    auto v_frag = [&](int s, int dt) __attribute__((always_inline)) {
      const int col = (((dt ^ v_swz) & (CH / 2 - 1)) << 5);  // swizzled 32-byte column block of d tile dt
      const lds_char *src = vbuf + v_lane_off + 32 * s * ROW_BYTES + col;
      const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3))) *)src);
      const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
          (s16x4 __attribute__((address_space(3))) *)(src + 16 * ROW_BYTES));
      const uint2 lo2 = __builtin_bit_cast(uint2, lo), hi2 = __builtin_bit_cast(uint2, hi);
      return vec16{{lo2.x, lo2.y, hi2.x, hi2.y}};  // the two 64-bit results are the operand as is
    };
    auto pv_slab = [&](int s) __attribute__((always_inline)) {
      constexpr int VAHEAD = 2;  // V fragments are read two d tiles ahead of their use
      vec16 vf[VAHEAD];
#pragma unroll
      for (int dt = 0; dt < VAHEAD; ++dt) vf[dt] = v_frag(s, dt);
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) {
#pragma unroll
        for (int qt = 0; qt < NQA; ++qt) o_acc[qt][dt] = M::run(vf[dt % VAHEAD], pf[qt][s], o_acc[qt][dt]);
        if (dt + VAHEAD < DT) vf[dt % VAHEAD] = v_frag(s, dt + VAHEAD);
      }
    };
    softmax_probs_slab<M, 0, NQA>(s_acc, m_run, l_acc, pf, ones, c);
    copy_point(3);
    __builtin_amdgcn_s_setprio(1);
    pv_slab(0);
    softmax_probs_slab<M, 1, NQA>(s_acc, m_run, l_acc, pf, ones, c);
    pv_slab(1);
    __builtin_amdgcn_s_setprio(0);
  };

  // ---- the part, in stretches of at most kWideTableTiles key tiles ------------------------------------------
  for (int seg0 = t_begin; seg0 < t_end; seg0 += kWideTableTiles) {
    const int seg1 = seg0 + kWideTableTiles < t_end ? seg0 + kWideTableTiles : t_end;
    if (seg0 != t_begin) __syncthreads();  // the previous stretch's last tile and table entries are still being read
    // slots of the stretch's keys; -1 marks a key past the end of its range or a slot outside the cache
    for (int i = tid; i < (seg1 - seg0) * BN; i += kWideThreads) {
      const TileRange tr = tile_range_of(seg0 + i / BN, tiles_a, shared_len, kv_len, BN);
      const int n = tr.n0 + i % BN;
      int slot = -1;
      if (n < tr.n_end) {
        slot = p.slot_map[kv_begin + n];
        if ((uint32_t)slot >= slot_limit) slot = -1;
      }
      lds_tbl[i] = slot;
    }
    __syncthreads();

    // this lane's table entries of tile u, and whether all rows of the wave's share exist
    auto tile_slots = [&](int u, int (&slots)[NI]) __attribute__((always_inline)) {
      bool present = true;
#pragma unroll
      for (int i = 0; i < NI; ++i) {
        slots[i] = lds_tbl[(u - seg0) * BN + dma_row0 + i * RPI];
        present &= slots[i] >= 0;
      }
      return __builtin_amdgcn_ballot_w64(!present) == 0;
    };
    auto stage_of = [&](int t) __attribute__((always_inline)) {
      return lds_ring + ((t - seg0) & (kWideStages - 1)) * STAGE_BYTES;
    };

    // prologue: the first three tiles of the stretch go out at once
    for (int u = seg0; u < seg1 && u < seg0 + kWideAhead; ++u) {
      int slots[NI];
      const bool all_present = tile_slots(u, slots);
#pragma unroll
      for (int cc = 0; cc < COPIES; ++cc) issue_copy(cc, stage_of(u), slots, all_present);
    }
    for (int t = seg0; t < seg1; ++t) {
      // this wave's copies of tile t have landed when at most the copies of the newer tiles are outstanding
      const int newer = seg1 - 1 - t < kWideAhead - 1 ? seg1 - 1 - t : kWideAhead - 1;
      if (newer >= 2) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * COPIES) : "memory");
      else if (newer == 1) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(COPIES) : "memory");
      else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      __syncthreads();  // ... and everybody else's; the buffer of tile t - 1 is no longer being read
      const int u = t + kWideAhead;
      int nslots[NI] = {};
      bool stepped = false;
      if (u < seg1) {
        stepped = tile_slots(u, nslots);
        if (!stepped) {
#pragma unroll
          for (int cc = 0; cc < COPIES; ++cc) issue_copy(cc, stage_of(u), nslots, false);
        }
      }
      if (MODE == MODE_QUERY_SIDE && t == tiles_a && t > t_begin) load_q(false);  // shared keys done: back to q
      const TileRange tr = tile_range_of(t, tiles_a, shared_len, kv_len, BN);
      if (nq_active == 2) {
        compute.template operator()<2>(stage_of(t), tr.n_end - tr.n0, stepped, stage_of(u), nslots);
      } else if (nq_active == 1) {
        compute.template operator()<1>(stage_of(t), tr.n_end - tr.n0, stepped, stage_of(u), nslots);
      } else if (stepped) {  // a wave without query rows only helps with the copies
#pragma unroll
        for (int cc = 0; cc < COPIES; ++cc) issue_copy(cc, stage_of(u), nslots, true);
      }
    }
  }
  __syncthreads();  // every wave is done reading the ring

  // ---- a unit dealt to several workgroups: leave the partial state, the last one to arrive merges ----------
  const int nparts = lds_uniform(entry + kPartNParts);
  if (nparts > 1) {
    const int part = lds_uniform(entry + kPartIndex), first_gid = lds_uniform(entry + kPartFirstGid);
    char *const ws_slots = reinterpret_cast<char *>(lds_uniform64(lds_par + kParSlots));
    int32_t *const ws_counters = reinterpret_cast<int32_t *>(lds_uniform64(lds_par + kParCounters));
    char *slot = ws_slots + (int64_t)(2 * (first_gid + part) + (part == 0 ? 1 : 0)) * kWideSlotBytes;
#pragma unroll
    for (int qt = 0; qt < NQ16; ++qt)
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
        store_f32x4_agent(slot + ((qt * DT + dt) * kWideThreads + tid) * 16, o_acc[qt][dt]);
    float *ml = reinterpret_cast<float *>(slot + kWideAccBytes);
#pragma unroll
    for (int qt = 0; qt < NQ16; ++qt) {
      store_f32_agent(ml + (2 * qt) * kWideThreads + tid, m_run[qt]);
      store_f32_agent(ml + (2 * qt + 1) * kWideThreads + tid, l_acc[qt][0]);
    }
    // the write-through stores above have been acknowledged before this part counts as arrived
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (tid == 0)
      *lds_flag = __hip_atomic_fetch_add(ws_counters + first_gid, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    if (*lds_flag != nparts - 1) return;  // another part is still at work: it will finish the unit
    if (tid == 0) __hip_atomic_store(ws_counters + first_gid, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    // The acquire drops whatever this XCD's L2 still holds of the slots from earlier calls.
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
    float l_fin[NQ16];
    if (nparts == 2) {
      // Two parts (the usual cut): this part's state is still in registers and the sum of two terms has no
      // order, so only the other part's slot is read, all of it in one batch of loads.
      const char *src = ws_slots + (int64_t)(2 * (first_gid + 1 - part) + (part == 1 ? 1 : 0)) * kWideSlotBytes;
      const float *mlp = reinterpret_cast<const float *>(src + kWideAccBytes);
      f32x4 other[NQ16][DT];
      float mo[NQ16], lo[NQ16];
#pragma unroll
      for (int qt = 0; qt < NQ16; ++qt) {
        mo[qt] = mlp[(2 * qt) * kWideThreads + tid];
        lo[qt] = mlp[(2 * qt + 1) * kWideThreads + tid];
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
          other[qt][dt] = *reinterpret_cast<const f32x4 *>(src + ((qt * DT + dt) * kWideThreads + tid) * 16);
      }
      {
        // products rounded before the sum (no fused multiply-add): only then is a*x + b*y the same as b*y + a*x
#pragma clang fp contract(off)
#pragma unroll
        for (int qt = 0; qt < NQ16; ++qt) {
          const float m_fin = fmaxf(m_run[qt], mo[qt]);
          const float a_own = m_run[qt] == -INFINITY ? 0.0f : __builtin_amdgcn_exp2f(m_run[qt] - m_fin);
          const float a_oth = mo[qt] == -INFINITY ? 0.0f : __builtin_amdgcn_exp2f(mo[qt] - m_fin);
          l_fin[qt] = l_acc[qt][0] * a_own + lo[qt] * a_oth;
#pragma unroll
          for (int dt = 0; dt < DT; ++dt) o_acc[qt][dt] = o_acc[qt][dt] * a_own + other[qt][dt] * a_oth;
        }
      }
    } else {
      // More parts: in part order from the slots (this part's own included), so the sum has one fixed order
      // whoever arrives last.
      float m_fin[NQ16];
#pragma unroll
      for (int qt = 0; qt < NQ16; ++qt) { m_fin[qt] = -INFINITY; l_fin[qt] = 0.0f; }
      for (int pp = 0; pp < nparts; ++pp) {
        const float *mlp = reinterpret_cast<const float *>(
            ws_slots + (int64_t)(2 * (first_gid + pp) + (pp == 0 ? 1 : 0)) * kWideSlotBytes + kWideAccBytes);
#pragma unroll
        for (int qt = 0; qt < NQ16; ++qt) m_fin[qt] = fmaxf(m_fin[qt], mlp[(2 * qt) * kWideThreads + tid]);
      }
#pragma unroll
      for (int qt = 0; qt < NQ16; ++qt)
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) o_acc[qt][dt] = f32x4{0, 0, 0, 0};
      for (int pp = 0; pp < nparts; ++pp) {
        const char *src = ws_slots + (int64_t)(2 * (first_gid + pp) + (pp == 0 ? 1 : 0)) * kWideSlotBytes;
        const float *mlp = reinterpret_cast<const float *>(src + kWideAccBytes);
#pragma unroll
        for (int qt = 0; qt < NQ16; ++qt) {
          const float mp = mlp[(2 * qt) * kWideThreads + tid];
          const float lp = mlp[(2 * qt + 1) * kWideThreads + tid];
          const float a = mp == -INFINITY ? 0.0f : __builtin_amdgcn_exp2f(mp - m_fin[qt]);
          l_fin[qt] += lp * a;
#pragma unroll
          for (int dt = 0; dt < DT; ++dt)
            o_acc[qt][dt] += *reinterpret_cast<const f32x4 *>(src + ((qt * DT + dt) * kWideThreads + tid) * 16) * a;
        }
      }
    }
#pragma unroll
    for (int qt = 0; qt < NQ16; ++qt) l_acc[qt][0] = l_fin[qt];
  }

  // ---- epilogue: normalise, transpose through LDS, store whole 16-byte chunks ------------------------------
  // Lane layout of O^T (query li, features 16*dt + 4*lg .. +4) would give 8-byte stores scattered over 16 rows;
  // staging the wave's 32 x D tile in LDS (rows padded to D*2 + 16 bytes against bank conflicts) lets 16
  // consecutive lanes write one full output row.
  {
    const int64_t o_token_bytes = lds_uniform64(lds_par + kParOutTokenBytes);
    char *out_base = reinterpret_cast<char *>(lds_uniform64(lds_par + kParOut)) +
                     (int64_t)lds_uniform(entry + kPartQBegin) * o_token_bytes +
                     (int64_t)lds_uniform(entry + kPartHead) * lds_uniform64(lds_par + kParOutHeadBytes);
    const int q_len_o = lds_uniform(entry + kPartQLen), q_tile0_o = lds_uniform(entry + kPartQTile0);
    constexpr int OPITCH = ROW_BYTES + 16;
    static_assert(kWideWaves * 32 * OPITCH <= kWideStages * STAGE_BYTES, "output staging must fit the ring");
    lds_char *stage = lds_ring + wave * (32 * OPITCH);
#pragma unroll
    for (int qt = 0; qt < NQ16; ++qt) {
      const float l = l_acc[qt][0];
      const float inv = l > 0.0f ? 1.0f / l : 1.0f;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) {
        lds_store8(stage + (qt * 16 + li) * OPITCH + (16 * dt + 4 * lg) * 2,
                   M::pack2(o_acc[qt][dt][0] * inv, o_acc[qt][dt][1] * inv),
                   M::pack2(o_acc[qt][dt][2] * inv, o_acc[qt][dt][3] * inv));
      }
    }
    // same wave wrote and reads: LDS accesses of one wave are ordered, no barrier needed
    constexpr int ROWS_PER_PASS = 64 / CH;
#pragma unroll
    for (int r0 = 0; r0 < 32; r0 += ROWS_PER_PASS) {
      const int r = r0 + lane / CH;
      const int qr = q_tile0_o + 16 * (wave + kWideWaves * (r >> 4)) + (r & 15);
      if (qr < q_len_o) {
        const vec16 v = lds_load16(stage + r * OPITCH + (lane % CH) * 16);
        store16(out_base + (int64_t)qr * o_token_bytes + (lane % CH) * 16, v);
      }
    }
  }
}

// Head groups and XCDs: consecutive block indices go to different XCDs (index mod 8), each with its own L2.
// With H_kv a multiple of 8 every XCD is a group of its own and owns H_kv / 8 KV heads; with H_kv = 1, 2 or 4,
// 8 / H_kv XCDs form the group of one KV head and their workgroups interleave on its timeline; otherwise all
// workgroups share one timeline over all heads.  Timeline of a group: requests in index order; per request the
// 256-row query tiles in order; per tile the heads of the group.  Tile t of a unit at position P starts at
// P + kUnit + t * c and belongs to the workgroup whose stretch contains that start.
constexpr int kPlanParts = 32;    // parts planned at a time

// The walk over the timeline, resumable: where the next unit starts and which one it is.
struct WideWalk {
  int64_t pos;   // timeline position of unit (b, j, e)
  int b, j, e;   // request, 256-row query tile, head of the group; b >= B: nothing left
};

template <int DTYPE, int D, int MODE>
__global__ __launch_bounds__(kWideThreads, 1) void varlen_attn_wide_kernel(AttnParams p) {
  constexpr int STAGE_BYTES = 2 * 64 * D * 2;
  constexpr int RING_BYTES = kWideStages * STAGE_BYTES, TABLE_BYTES = kWideTableTiles * 64 * 4;
  // one block, so that the ring keeps its 1 KiB alignment (the swizzle that makes the fragment reads
  // conflict-free counts on it); the slot table, the flag word and the plan sit behind it
  __shared__ __attribute__((aligned(1024))) char lds[RING_BYTES + TABLE_BYTES + 16 + (kPlanParts * kPlanInts + 32) * 4];
  lds_char *const lds_ring = (lds_char *)lds;
  lds_int *const lds_tbl = (lds_int *)(lds_ring + RING_BYTES);
  lds_int *const lds_flag = (lds_int *)(lds_ring + RING_BYTES + TABLE_BYTES);
  lds_int *const lds_plan = (lds_int *)(lds_ring + RING_BYTES + TABLE_BYTES + 16);  // [0]: parts, [1]: more to come,
  lds_int *const lds_walk = lds_plan + 2;                                           // [2..8): walk state, [16..): parts
  lds_int *const lds_par = lds_plan + 16;    // [16..26): output and workspace pointers
  lds_int *const lds_parts = lds_plan + 32;

  // ---- which stretch of which timeline is this workgroup's? -----------------------------------------
  // (This block and the planning block below keep their many scalars to themselves: while a unit is being
  // computed only a loop counter is live.  Kept alive across the key loop they push it over the scalar-register
  // budget, and the instruction scheduler answers excess pressure by giving up the early issue of the fragment
  // reads that the loop depends on.)
  if (threadIdx.x < 64) {  // wave 0 lays the workgroup's stretch out; everybody reads it from LDS
    const int lane = threadIdx.x;
    const int xcd = blockIdx.x & 7, idx = blockIdx.x >> 3;
    const int n_super = p.H_kv % 8 == 0 ? 8 : (8 % p.H_kv == 0 ? p.H_kv : 1);
    const int xcds_per_super = 8 / n_super;
    const int k = idx * xcds_per_super + xcd % xcds_per_super;   // this workgroup's index on the timeline
    const int wgs = (gridDim.x >> 3) * xcds_per_super;           // workgroups on the timeline
    const int hs = p.H / n_super;                                // heads on the timeline
    int64_t total = 0;
    for (int b0 = 0; b0 < p.B; b0 += 64) {
      int64_t w = b0 + lane < p.B ? wide_request_weight(wide_request<MODE>(p, b0 + lane)) : 0;
#pragma unroll
      for (int d = 1; d < 64; d <<= 1) w += __shfl_xor(w, d);
      total += w;
    }
    total = uniform64(total) * hs;
    int64_t stretch = (total + wgs - 1) / wgs;
    if (stretch < kMinStretch) stretch = kMinStretch;  // small calls run on fewer workgroups, not on slivers
    const int64_t lo = (int64_t)k * stretch;
    WideWalk w{0, p.B, 0, 0};
    if (lo < total) {
      // the request whose units contain position lo, and where it starts
      int b = 0;
      int64_t pos = 0, base = 0;
      for (int b0 = 0; b0 < p.B; b0 += 64) {
        const int64_t wt = b0 + lane < p.B ? wide_request_weight(wide_request<MODE>(p, b0 + lane)) * hs : 0;
        int64_t incl = wt;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
          const int64_t up = __shfl_up(incl, d);
          if (lane >= d) incl += up;
        }
        const uint64_t hit = __builtin_amdgcn_ballot_w64(base + incl > lo);
        if (hit != 0) {
          const int src = __builtin_ctzll(hit);
          b = b0 + src;
          pos = base + __shfl(incl - wt, src);
          break;
        }
        base += __shfl(incl, 63);
      }
      b = __builtin_amdgcn_readfirstlane(b);
      pos = uniform64(pos);
      const WideRequest r = wide_request<MODE>(p, b);
      // unit (query tile j, head e of the group) of request b that contains lo; pos becomes its start
      const int64_t off = lo - pos;
      const int64_t full_span = (int64_t)(r.nt - 1) * hs * r.w_full;
      int64_t u;
      if (off < full_span) {
        u = off / r.w_full;
        pos += u * r.w_full;
      } else {
        const int64_t u2 = (off - full_span) / r.w_last;
        u = (int64_t)(r.nt - 1) * hs + u2;
        pos += full_span + u2 * r.w_last;
      }
      w = WideWalk{pos, b, (int)(u / hs), (int)(u % hs)};
    }
    if (lane == 0) {
      auto put64 = [&](int i, uint64_t v) __attribute__((always_inline)) {
        lds_par[i] = (int)(uint32_t)v;
        lds_par[i + 1] = (int)(uint32_t)(v >> 32);
      };
      put64(kParOut, (uint64_t)(uintptr_t)p.out);
      put64(kParOutTokenBytes, (uint64_t)p.o_token_bytes);
      put64(kParOutHeadBytes, (uint64_t)p.o_head_bytes);
      put64(kParSlots, (uint64_t)(uintptr_t)p.ws_slots);
      put64(kParCounters, (uint64_t)(uintptr_t)p.ws_counters);
      lds_walk[0] = (int)(uint32_t)(uint64_t)w.pos;
      lds_walk[1] = (int)(uint32_t)((uint64_t)w.pos >> 32);
      lds_walk[2] = w.b; lds_walk[3] = w.j; lds_walk[4] = w.e;
      lds_walk[5] = (int)(uint32_t)(uint64_t)stretch;
      lds_walk[6] = (int)(uint32_t)((uint64_t)stretch >> 32);
    }
  }

  while (true) {
    __syncthreads();  // the walk state is in place; nobody reads the previous plan any more
    // ---- plan: the next parts of the stretch, at most kPlanParts -----------------------------------------
    if (threadIdx.x < 64) {
      const int xcd = blockIdx.x & 7, idx = blockIdx.x >> 3;
      const int n_super = p.H_kv % 8 == 0 ? 8 : (8 % p.H_kv == 0 ? p.H_kv : 1);
      const int xcds_per_super = 8 / n_super;
      const int super = xcd / xcds_per_super;
      const int k = idx * xcds_per_super + xcd % xcds_per_super;
      const int wgs = (gridDim.x >> 3) * xcds_per_super;
      const int hs = p.H / n_super;
      const bool split = p.ws_slots != nullptr;
      auto rd = [&](int i) __attribute__((always_inline)) { return __builtin_amdgcn_readfirstlane(lds_walk[i]); };
      int64_t pos = (int64_t)(((uint64_t)(uint32_t)rd(1) << 32) | (uint32_t)rd(0));
      int b = rd(2), j = rd(3), e = rd(4);
      const int64_t stretch = (int64_t)(((uint64_t)(uint32_t)rd(6) << 32) | (uint32_t)rd(5));
      const int64_t lo = (int64_t)k * stretch, hi = lo + stretch;  // units end at or before the total
      int n = 0, more = 0;
      if (b < p.B) {
        WideRequest r = wide_request<MODE>(p, b);
        while (true) {
          const bool last_tile = j == r.nt - 1;
          const int q_tile0 = j * kWideRows;
          const int c = last_tile ? wide_tile_cost(r.q_len - q_tile0) : 20;
          const int64_t first = pos + kUnit;  // start of the unit's first key tile
          if (first >= hi) { b = p.B; break; }  // everything from here on belongs to later workgroups
          if (n == kPlanParts) { more = 1; break; }
          int t0, t1, nparts = 1, part = 0, first_wg = k;
          if (split) {
            t0 = first >= lo ? 0 : (int)((lo - first + c - 1) / c);
            const int64_t upto = (hi - first + c - 1) / c;
            t1 = upto < r.kt ? (int)upto : r.kt;
            first_wg = (int)(first / stretch);
            nparts = (int)((first + (int64_t)(r.kt - 1) * c) / stretch) - first_wg + 1;
            part = k - first_wg;
          } else {  // no workspace: units are dealt whole, to the workgroup that holds their first tile
            t0 = 0;
            t1 = first >= lo ? r.kt : 0;
          }
          if (t0 < t1) {
            if (threadIdx.x == 0) {
              lds_int *dst = lds_parts + n * kPlanInts;
              dst[kPartB] = b; dst[kPartQTile0] = q_tile0; dst[kPartHead] = super * hs + e;
              dst[kPartTBegin] = t0; dst[kPartTEnd] = t1; dst[kPartNParts] = nparts; dst[kPartIndex] = part;
              dst[kPartFirstGid] = super * wgs + first_wg; dst[kPartQBegin] = r.q_begin; dst[kPartQLen] = r.q_len;
            }
            ++n;
          }
          pos += last_tile ? r.w_last : r.w_full;
          if (++e == hs) {
            e = 0;
            if (++j == r.nt) {
              j = 0;
              do {
                if (++b < p.B) r = wide_request<MODE>(p, b);
              } while (b < p.B && r.nt == 0);
              if (b >= p.B) break;
            }
          }
        }
      }
      if (threadIdx.x == 0) {
        lds_plan[0] = n; lds_plan[1] = more;
        lds_walk[0] = (int)(uint32_t)(uint64_t)pos;
        lds_walk[1] = (int)(uint32_t)((uint64_t)pos >> 32);
        lds_walk[2] = b; lds_walk[3] = j; lds_walk[4] = e;
      }
    }
    __syncthreads();
    const int n_parts = __builtin_amdgcn_readfirstlane(lds_plan[0]);
    for (int i = 0; i < n_parts; ++i) {
      attn_wide_part<DTYPE, D, MODE>(p, lds_ring, lds_tbl, lds_flag, lds_parts + i * kPlanInts, lds_par);
    }
    if (__builtin_amdgcn_readfirstlane(lds_plan[1]) == 0) break;
  }
}

}  // namespace acache

using namespace acache;

// Workgroups of the persistent grid on the current device: one per CU, a multiple of 8 (one share per XCD).
static int wide_grid_of_current_device(int *wgs) {
  static int cached[64] = {0};
  int dev = 0;
  hipError_t err = hipGetDevice(&dev);
  if (err != hipSuccess) return fail((int)err, "varlen_attn: hipGetDevice: %s", hipGetErrorString(err));
  const bool cacheable = dev >= 0 && dev < 64;
  if (!cacheable || cached[dev] == 0) {
    int cus = 0;
    err = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
    if (err != hipSuccess || cus <= 0)
      return fail(err != hipSuccess ? (int)err : ACACHE_E_RANGE, "varlen_attn: cannot read the CU count");
    int g = cus / 8 * 8;
    if (g < 8) g = 8;
    if (!cacheable) { *wgs = g; return 0; }
    cached[dev] = g;
  }
  *wgs = cached[dev];
  return 0;
}

static int64_t wide_counter_bytes(int wgs) {
  return ((int64_t)wgs * 4 + kWideCounterAlign - 1) / kWideCounterAlign * kWideCounterAlign;
}

namespace acache {

int64_t attn_wide_workspace_bytes() {
  int wgs = 0;
  if (wide_grid_of_current_device(&wgs)) return -1;
  return wide_counter_bytes(wgs) + (int64_t)2 * wgs * kWideSlotBytes;
}

// Launch the wide kernel (head_dim 64 / 128, plain or query-side mode).  workspace may be NULL or too small:
// units are then dealt whole.
int launch_attn_wide(const AttnParams &p0, int dtype, int D, int mode, void *workspace, int64_t workspace_bytes,
                     hipStream_t stream) {
  AttnParams p = p0;
  int wgs = 0;
  const int rc = wide_grid_of_current_device(&wgs);
  if (rc) return rc;
  p.ws_counters = nullptr;
  p.ws_slots = nullptr;
  if (workspace && workspace_bytes >= wide_counter_bytes(wgs) + (int64_t)2 * wgs * kWideSlotBytes) {
    p.ws_counters = (int32_t *)workspace;
    p.ws_slots = (char *)workspace + wide_counter_bytes(wgs);
  }
#define ACACHE_WIDE(DT, DD, MM)                                                                                   \
  if (dtype == DT && D == DD && mode == MM) {                                                                     \
    hipLaunchKernelGGL((varlen_attn_wide_kernel<DT, DD, MM>), dim3((unsigned)wgs), dim3(kWideThreads), 0, stream, p); \
    return launch_status("varlen_attn_wide_kernel");                                                              \
  }
  ACACHE_WIDE(ACACHE_BF16, 128, MODE_PLAIN)
  ACACHE_WIDE(ACACHE_BF16, 128, MODE_QUERY_SIDE)
  ACACHE_WIDE(ACACHE_BF16, 64, MODE_PLAIN)
  ACACHE_WIDE(ACACHE_BF16, 64, MODE_QUERY_SIDE)
  ACACHE_WIDE(ACACHE_F16, 128, MODE_PLAIN)
  ACACHE_WIDE(ACACHE_F16, 128, MODE_QUERY_SIDE)
  ACACHE_WIDE(ACACHE_F16, 64, MODE_PLAIN)
  ACACHE_WIDE(ACACHE_F16, 64, MODE_QUERY_SIDE)
#undef ACACHE_WIDE
  return fail(ACACHE_E_SHAPE, "varlen_attn (wide): unsupported dtype / head_dim / mode");
}

}  // namespace acache
