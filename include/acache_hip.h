/*
 * libacache_hip — C ABI of the MI355X (gfx950) affix-KV reuse kernels.
 *
 * The reference (sands-lab/ACache) has no C ABI: its boundary for this path is a
 * set of Python callables that launch Triton kernels.  Each entry point below
 * replaces one of those launches; the citation names the reference callable
 * (path relative to the reference tree) whose arithmetic it reproduces.
 *
 * Conventions shared by every entry point
 *   - all data pointers are DEVICE pointers owned by the caller; nothing is
 *     allocated, freed or retained by the library (entry points that need scratch
 *     memory take it as a workspace argument; acache_affix_importance_noalloc is the
 *     one exception and says so);
 *   - work is enqueued on `stream` (a hipStream_t passed as void*, NULL = the
 *     default stream) and the call returns without synchronising;
 *   - return value: 0 = enqueued; < 0 = argument error (ACACHE_E_*), nothing was
 *     launched; > 0 = the hipError_t reported by the launch;
 *   - acache_last_error() returns a thread-local, human readable description of
 *     the most recent non-zero return on the calling thread;
 *   - calls are re-entrant across distinct streams; no global mutable state
 *     (except the built-in scratch of acache_affix_importance_noalloc);
 *   - strides and offsets are counted in ELEMENTS of `dtype`, never bytes;
 *   - slot = block_id * cache_block_size + offset_in_block: an index into the
 *     cache viewed as [num_slots, H_kv, D] (per layer).
 */
#ifndef ACACHE_HIP_H
#define ACACHE_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ACACHE_ABI_VERSION 4

/* element types of K/V/Q payloads */
#define ACACHE_BF16 0
#define ACACHE_F16  1
#define ACACHE_F32  2

/* argument errors */
#define ACACHE_E_NULL      -1  /* a required pointer is NULL                         */
#define ACACHE_E_DTYPE     -2  /* dtype not supported by this entry point            */
#define ACACHE_E_SHAPE     -3  /* head_dim / head counts / sizes not supported       */
#define ACACHE_E_RANGE     -4  /* slot range, shift or table rows out of range       */
#define ACACHE_E_OVERLAP   -5  /* source and destination rows overlap                */
#define ACACHE_E_ALIGN     -6  /* pointer or stride breaks the 16-byte alignment rule */
#define ACACHE_E_MODE      -7  /* inconsistent relocation arguments                  */

int acache_abi_version(void);
const char *acache_last_error(void);

/*
 * Relocate + RoPE re-rotate + gather into the packed varlen layout.
 *
 *   for l < L, t < T, h < H_kv:
 *     out_k[l, t, h, :] = rotate(k_cache[l, slot_map[t], h, :], delta[t])
 *     out_v[l, t, h, :] =        v_cache[l, slot_map[t], h, :]
 *   rotate(x, d) = x * cos[|d|] + rot_half(x) * sgn(d) * sin[|d|],
 *   rot_half(x)  = cat(-x[D/2:], x[:D/2]); fp32 multiply, multiply, add (each
 *   rounded, no fused multiply-add), one rounding to `dtype` on store.
 *   Rows with delta[t] == 0 (or delta == NULL) are bit copies.
 *
 * This is the un-fused form of the reference's key-side relocation inside
 * attention (nano-vdllm/model/acache_attention.py:475-497: gather by
 * read_slot_map, rotate rows of shared slots by delta = n - slot with the
 * sin sign rule of line 496) and of the dense-cache slice copy of the HF path
 * (llada/generate_ACache.py:501-512).
 *
 * Out-of-range inputs never fault: a row whose slot is outside [0, num_slots)
 * or whose |delta| >= rope_rows is written as zeros (K and V).
 *
 * rope_cos / rope_sin: fp32 [rope_rows, D] contiguous, may be NULL iff delta is NULL.
 * D: half a row must be a whole number of 16-byte chunks (bf16 / f16: a multiple of 16,
 * f32: a multiple of 8); 128 and 64 take the tuned kernel.
 * cache_layer_stride / out_layer_stride: elements between consecutive layers.
 * Token rows are contiguous: [.., H_kv, D] with strides (H_kv*D, D, 1).
 */
int acache_relocate_rope_gather(
    void *out_k, void *out_v,
    const void *k_cache, const void *v_cache,
    const int32_t *slot_map, const int32_t *delta,
    const float *rope_cos, const float *rope_sin,
    int64_t T, int32_t L, int32_t H_kv, int32_t D, int32_t dtype,
    int64_t num_slots, int32_t rope_rows,
    int64_t cache_layer_stride, int64_t out_layer_stride,
    void *stream);

/*
 * In-place materialisation of a relocated affix copy, all layers in one launch.
 *
 *   for l < L, t < affix_len, h < H_kv:
 *     k_cache[l, dst_slot + t, h, :] = rotate(k_cache[l, t, h, :], affix_shift)
 *     v_cache[l, dst_slot + t, h, :] =        v_cache[l, t, h, :]
 *
 * Replaces materialize_relocated_affix and its per-layer launch loop
 * (nano-vdllm/model/acache_attention.py:6-128; caller
 * nano-vdllm/model_runner.py:314-341).  [0, affix_len) and
 * [dst_slot, dst_slot + affix_len) must not overlap (ACACHE_E_OVERLAP) and must
 * lie inside [0, num_slots); |affix_shift| < rope_rows (ACACHE_E_RANGE).
 */
int acache_materialize_relocated_affix(
    void *k_cache, void *v_cache,
    const float *rope_cos, const float *rope_sin,
    int64_t dst_slot, int64_t affix_len, int32_t affix_shift,
    int32_t L, int32_t H_kv, int32_t D, int32_t dtype,
    int64_t num_slots, int32_t rope_rows, int64_t cache_layer_stride,
    void *stream);

/*
 * Scatter freshly computed K/V rows into the paged cache.
 *
 *   for l < L, i < N: if slot_map[i] != -1:
 *     k_cache[l, slot_map[i], :, :] = key[l, i, :, :]   (same for value)
 *
 * Replaces store_kvcache / store_kvcache_kernel
 * (nano-vdllm/model/attention.py:11-41), which the reference launches once per
 * layer (L = 1 here reproduces that call).  Rows are bit copies.  A slot outside
 * [-1, num_slots) is skipped like -1.  Duplicate slots inside one call are
 * undefined (as in the reference).
 * key_token_stride / value_token_stride: elements between consecutive tokens
 * of the source (>= H_kv*D, the reference's key.stride(0)); src_layer_stride:
 * elements between layers of the source (ignored when L == 1).
 */
int acache_kv_scatter(
    void *k_cache, void *v_cache,
    const void *key, const void *value,
    const int32_t *slot_map,
    int64_t N, int32_t L, int32_t H_kv, int32_t D, int32_t dtype,
    int64_t num_slots,
    int64_t key_token_stride, int64_t value_token_stride,
    int64_t src_layer_stride, int64_t cache_layer_stride,
    void *stream);

/*
 * RoPE on freshly projected q / k rows, fused with the scatter of k / v into the
 * paged cache of one layer: the step in front of attention.
 *
 *   for i < N, with p = positions[i]:
 *     q[i, h, :]  = rope(q[i, h, :], p)            for h < H      (in place)
 *     k[i, h, :]  = rope(k[i, h, :], p)            for h < H_kv   (in place)
 *     if slot_map[i] >= 0:
 *       k_cache[slot_map[i], :, :] = k[i, :, :]   (the rotated rows)
 *       v_cache[slot_map[i], :, :] = v[i, :, :]
 *   rope(x, p) = x * cos[p] + rot_half(x) * sin[p] in fp32, products and sum
 *   rounded separately, one rounding to `dtype`.
 *
 * Replaces the rotary application of the model's attention block
 * (nano-vdllm/model/modeling_llada.py:412-453: q and k up-cast, rotated with the
 * cat(freqs, freqs) tables at the given position ids, cast back) followed by
 * store_kvcache (nano-vdllm/model/attention.py:34-41, called at line 72); one
 * launch instead of the reference's elementwise chain plus the scatter kernel.
 *
 * slot_map may be NULL (no cache write; v and the caches are then unused).  A slot
 * outside [0, num_slots) is skipped like -1; a position outside [0, rope_rows)
 * leaves the row unrotated.  q / k / v: [N, heads, D] with the given token
 * strides (heads contiguous, so the three may be views of one fused projection).
 * D: half a row must be a whole number of 16-byte chunks (128 and 64 take the tuned kernel).
 */
int acache_rope_qk_scatter(
    void *q, void *k, const void *v, void *k_cache, void *v_cache,
    const int64_t *positions, const int32_t *slot_map,
    const float *rope_cos, const float *rope_sin, int32_t rope_rows,
    int64_t N, int32_t H, int32_t H_kv, int32_t D, int32_t dtype, int64_t num_slots,
    int64_t q_token_stride, int64_t k_token_stride, int64_t v_token_stride,
    void *stream);

/*
 * Affix importance for anchor selection: attention of each request's [MASK] queries
 * to the cached affix keys, soft-maxed over the affix keys only, summed over the
 * mask queries and the heads of one layer and ADDED to importance[b, :].
 *
 *   for b < B, r in mask_rows[cu_mask[b] .. cu_mask[b+1]), h < H:
 *     w[a] = softmax_a( rot(q[r, h], -affix_shifts[b]) . k_cache[affix_slot0 + a, h / (H/H_kv)] * scale ), a < affix_len
 *     importance[b, a] += w[a]
 *   rot(q, -s) = q*cos[s] - rot_half(q)*sin[s] in fp32, rounded once to `dtype` (the query-side
 *   relocation of acache_varlen_attn); it equals q . rot(k, +s) before rounding.  fp32 scores and softmax.
 *
 * Replaces the per-request loop of the patched attention forward in
 * _compute_anchor_positions_batch (nano-vdllm/model_runner.py:730-773: rotary
 * re-application on the cached affix keys, matmul, softmax, two sums, add_), once
 * per layer; call it for every layer on the same importance buffer, then
 * acache_topk_anchors.  The reference evaluates matmul and softmax in the model
 * dtype and rounds the re-rotated keys to it; here scores and softmax are fp32 and the
 * rotation (and its rounding) sits on the queries, so every request reads the one
 * cached copy of the keys.  Deterministic: no atomics, fixed summation order.
 *
 * mask_rows are row indices into q ([total_q, H, D] with the given strides); an index outside
 * [0, total_q) is an absent query and adds nothing.  workspace:
 * device scratch of at least acache_affix_importance_workspace_bytes(total_mask_rows, B, H,
 * H_kv, D, affix_len, relocated = affix_shifts != NULL) bytes (row statistics, per-head
 * partial sums and the packed, counter-rotated copy of the mask queries,
 * passed between the launches), 16-byte aligned, owned by the caller.  max_mask_rows: an upper bound on
 * the mask rows of one request; a request whose cu_mask entries claim more rows than that, or more than
 * total_mask_rows leaves room for, is scored on the rows that fit (cu_mask is device memory the host does
 * not read).  D: a multiple of 16 up to 256; dtype bf16 or f16.
 */
int64_t acache_affix_importance_workspace_bytes(int64_t total_mask_rows, int32_t B, int32_t H, int32_t H_kv,
                                                int32_t D, int32_t affix_len, int32_t relocated);
int acache_affix_importance(
    float *importance, const void *q, const void *k_cache,
    const int32_t *mask_rows, const int32_t *cu_mask, const int32_t *affix_shifts,
    const float *rope_cos, const float *rope_sin, int32_t rope_rows, float scale,
    int32_t affix_len, int64_t affix_slot0, int32_t B, int64_t total_q, int64_t total_mask_rows,
    int32_t max_mask_rows, int32_t H, int32_t H_kv, int32_t D, int32_t dtype, int64_t num_slots,
    int64_t importance_stride, int64_t q_token_stride, int64_t q_head_stride,
    int64_t kv_slot_stride, int64_t kv_head_stride,
    void *workspace, int64_t workspace_bytes, void *stream);

/*
 * acache_affix_importance for callers that cannot allocate device memory.
 *
 * No counterpart in the reference.  It exists for callers that may not call hipMalloc (or
 * torch's allocator) around the probe: code under HIP graph capture, tight serving loops,
 * harnesses that forbid allocation.  Same arguments, arithmetic and results as
 * acache_affix_importance, bit for bit, minus the workspace: the scratch is a file-scope device
 * array of ACACHE_IMPORTANCE_SCRATCH_BYTES inside the library (one copy per GPU the library
 * runs on, held until the process ends; its address is looked up on the first call on each
 * device).  The call allocates and frees nothing.
 *
 * A call whose acache_affix_importance_workspace_bytes(...) exceeds the array is rejected with
 * ACACHE_E_SHAPE before anything is launched.  All calls on one GPU share that GPU's array:
 * calls that overlap in time on the same GPU (different streams or threads) race; serialise
 * them.  The current device must be the one `stream` belongs to.
 */
#define ACACHE_IMPORTANCE_SCRATCH_BYTES (40 << 20)
int64_t acache_affix_importance_noalloc_max_bytes(void);
int acache_affix_importance_noalloc(
    float *importance, const void *q, const void *k_cache,
    const int32_t *mask_rows, const int32_t *cu_mask, const int32_t *affix_shifts,
    const float *rope_cos, const float *rope_sin, int32_t rope_rows, float scale,
    int32_t affix_len, int64_t affix_slot0, int32_t B, int64_t total_q, int64_t total_mask_rows,
    int32_t max_mask_rows, int32_t H, int32_t H_kv, int32_t D, int32_t dtype, int64_t num_slots,
    int64_t importance_stride, int64_t q_token_stride, int64_t q_head_stride,
    int64_t kv_slot_stride, int64_t kv_head_stride, void *stream);

/*
 * Per-request top-k anchor selection over ragged fp32 influence scores.
 *
 *   request b owns scores[cu_affix[b] .. cu_affix[b+1]) and selects
 *   K_b = cu_k[b+1] - cu_k[b] indices: the first K_b under the order
 *   "higher score first, then lower index" (largest != 0) or
 *   "lower score first, then lower index" (largest == 0); they are written
 *   ASCENDING to out_idx[cu_k[b] .. cu_k[b+1]) with offsets[b] added
 *   (offsets may be NULL).
 *
 * Replaces torch.topk(...).indices.sort() at
 * nano-vdllm/model_runner.py:833-843, llada/generate_ACache.py:247-260 and
 * dream/generate_ACache.py:367-373.  torch leaves the order of equal scores
 * unspecified; this library fixes it to the lower index.  -0.0 equals +0.0;
 * NaN ranks above +inf (torch.topk's convention).  K_b is clamped to the
 * request's score count.  idx_bytes selects int32 (4) or int64 (8) output.
 */
int acache_topk_anchors(
    void *out_idx, const float *scores,
    const int32_t *cu_affix, const int32_t *cu_k, const int32_t *offsets,
    int32_t largest, int32_t B, int32_t idx_bytes,
    void *stream);

/*
 * Proposed token and its confidence per logits row (masked-diffusion transfer rule).
 *
 *   for r < R:
 *     t = picks ? picks[r] : argmax_v logits[r, v]          (first maximum)
 *     out_token[r] = t
 *     out_conf[r]  = exp(logits[r, t] - logsumexp_v logits[r, v])    in fp32
 *
 * Replaces the per-64-row loop of get_transfer_index
 * (nano-vdllm/model_runner.py:2279-2296: up-cast to fp32, gather of the chosen
 * logit, torch.logsumexp, exp) and the arg-max in front of it at temperature 0;
 * with temperature > 0 the caller draws the Gumbel arg-max itself and passes it
 * as `picks` (out_token may then be NULL).  The row is read once.
 * NaN: a NaN logit is never chosen as the arg-max (torch.argmax would return its
 * index) but it enters the sum, so the row's confidence is NaN and the caller's
 * `confidence >= threshold` test fails for it: on a row that holds a NaN this
 * entry point and the reference's torch formulation may name different tokens, and
 * neither commits one by threshold.  row_stride in elements, a multiple of 16 bytes.
 */
int acache_argmax_confidence(
    int64_t *out_token, float *out_conf, const void *logits, const int64_t *picks,
    int64_t R, int64_t V, int64_t row_stride, int32_t dtype, void *stream);

/*
 * The commit step behind it: write the accepted proposals into the working blocks.
 *
 *   for r < n, i < L (blocks, proposal: int64 [n, L]; confidence: fp32 [n, L]; all contiguous):
 *     committable[r, i] = blocks[r, i] == mask_id && proposal[r, i] != mask_id
 *     accept[r, i]      = committable[r, i] && confidence[r, i] >= threshold
 *     a row with committable positions and no accepted one accepts its most confident
 *     committable position (the first of equals)
 *     blocks[r, i] = proposal[r, i] where accepted; every other entry is left as it is
 *   *committed_rows += number of rows that accepted at least one position (atomic; the caller
 *   compares the counter before and after to learn whether the step made progress)
 *
 * Replaces the mask / threshold / forced-pick tensor operations of get_transfer_index and the
 * write of its picks into the working blocks (nano-vdllm/model_runner.py:2297-2314, 2262-2266)
 * by one launch, one wave per row.  Differs from the reference in the rule this library's host
 * documents: a position whose proposal is the mask token itself is never accepted (writing it
 * would change nothing, and as a forced pick it would repeat the same step for ever).
 * Confidences are expected to be numbers (a NaN is never accepted by threshold and is forced
 * only when it is the row's first committable position).
 */
int acache_commit_tokens(
    int64_t *blocks, const int64_t *proposal, const float *confidence, int32_t *committed_rows,
    int64_t n, int32_t L, int64_t mask_id, float threshold, void *stream);

/*
 * Expand per-request block tables into a flat slot map.
 *
 *   out_slots[cu_k[b] + n] = block_tables[b, n / block_size] * block_size + n % block_size
 *   for n < cu_k[b+1] - cu_k[b]
 *
 * The addressing rule of the reference's block-table attention kernels
 * (nano-vdllm/model/acache_attention.py:194-196, 295-297) and of
 * prepare_decoding (nano-vdllm/model_runner.py:1100-1110).  Table entries past
 * a request's last block (-1 padding) are never read.
 */
int acache_block_table_slots(
    int32_t *out_slots, const int32_t *block_tables, const int32_t *cu_k,
    int32_t B, int32_t max_blocks, int32_t block_size, int64_t total_k,
    void *stream);

/*
 * Slot layout of a batch of requests that reuse a shared affix (device-side form of
 * Sequence.finalize_slot_mapping, nano-vdllm/sequence.py:169-202, which the reference
 * evaluates per request in Python before prepare_caching_acache,
 * nano-vdllm/model_runner.py:1295-1471).
 *
 *   request b: tokens [0, len_b), affix [affix_start[b], affix_end[b]), anchors
 *   anchors[cu_anchor[b] .. cu_anchor[b+1]) (ascending positions inside the affix),
 *   private slot i = block_tables[b, i / block_size] * block_size + i % block_size.
 *   The first K_b private slots belong to the anchors in position order, the rest to
 *   the positions outside the affix in order.
 *     read_slots[cu_len[b] + pos] = private slot of pos            (anchor or non-affix)
 *                                 = shared_slot_offset + pos - affix_start[b]   (frozen affix)
 *     recompute_pos / recompute_slots[cu_rec[b] + j]: the recomputed positions of b in
 *     ascending order with their slots (K_b + len_b - affix_len_b entries).
 */
int acache_build_slot_layout(
    int32_t *read_slots, int32_t *recompute_pos, int32_t *recompute_slots,
    const int32_t *cu_len, const int32_t *cu_rec,
    const int32_t *affix_start, const int32_t *affix_end,
    const int32_t *cu_anchor, const int32_t *anchors,
    const int32_t *block_tables, int32_t B, int32_t max_blocks, int32_t block_size,
    int32_t shared_slot_offset, int64_t total_tokens, void *stream);

/*
 * Bidirectional variable-length attention reading K/V through a slot map.
 *
 *   per request b, head h (kv head = h / (H / H_kv)):
 *     K_b[n] = k_cache[slot_map[cu_k[b] + n], kv head],  V_b[n] likewise
 *     out[cu_q[b] + m, h] = softmax_n(q[cu_q[b] + m, h] . K_b[n] * scale) . V_b
 *   fp32 accumulation, probabilities rounded to `dtype` before the PV product,
 *   output rounded to `dtype`.  The scale is applied to the fp32 product, as the reference does
 *   (lines 439, 460, 499): scores of any magnitude keep the 2e-2 absolute bound on outputs that the
 *   parity tests hold this call to.
 *
 * Relocation modes (selected exactly as the reference wrapper does,
 * nano-vdllm/model/acache_attention.py:670-671):
 *   plain      : shared_prefix_len == 0 or affix_shifts == NULL
 *   key side   : affix_shifts != NULL, shared_kv_lens == NULL — rows with
 *                slot < shared_prefix_len are rotated by delta = n - slot
 *                (lines 480-497)
 *   query side : affix_shifts and shared_kv_lens given — the first
 *                shared_kv_lens[b] keys of request b are scored against
 *                q' = round(q*cos[s] - rot_half(q)*sin[s]), s = affix_shifts[b]
 *                (lines 399-469)
 * Replaces acache_attention / _acache_attention_kernel (lines 337-514, 643-738);
 * with a slot map from acache_block_table_slots it also replaces
 * baseline_ragged_attention and baseline_decode_attention (lines 131-334,
 * 525-640).  Unlike the reference, rows of requests with no keys are written
 * as zeros instead of being left uninitialised, and no host synchronisation is
 * needed: the grid is sized from total_q and B.
 *
 * Supported: D a multiple of 16 up to 256 (128 and 64 take the tuned kernels, every other
 * width a padded one, as the reference pads to the next power of two, lines 517-522),
 * dtype bf16 or f16, H % H_kv == 0, scale > 0 (ACACHE_E_RANGE otherwise).  A key whose
 * slot lies outside [0, num_slots) reads as a zero row.
 * q / out: [total_q, H, D] with given token and head strides (innermost 1).
 * k_cache / v_cache: [num_slots, H_kv, D] with given slot and head strides.
 * cu_q / cu_k are device memory and taken as given, as the reference takes its cu_seqlens:
 * non-decreasing prefix sums of B + 1 entries with cu_q[0] == cu_k[0] == 0, cu_q[B] == total_q and
 * cu_k[B] == total_k (the length of slot_map).  Slot values are checked per key, the prefix sums are not.
 *
 * Schedule (head_dim 64 / 128).  One workgroup of four waves per (request, 128-row query tile, head)
 * unit, two workgroups per CU, units handed out longest request first; K/V tiles of 64 keys reach LDS
 * through the copy engine.  In key-side mode the rows of a tile that lie in shared slots are re-rotated
 * in LDS after they land.  No workspace: the kernel allocates nothing and keeps no state between calls.
 *
 * acache_varlen_attn_planned is the same call with the order of the units given by the caller:
 * `plan` (device memory, 8-byte aligned, 2 * plan_blocks int32, written by
 * acache_varlen_attn_plan for the same cu_q, cu_k, H and H_kv) names the unit of every block of the
 * grid.  The hardware hands blocks out in index order, so with two or three units per workgroup
 * slot the order decides how evenly the slots finish; a plan packs them (measured on configs[3] of
 * the benchmark: 96 -> 87 us).  Results are bit-identical with and without a plan.  The kernel checks
 * every plan entry against B, H and cu_q: a plan made for other lengths can leave output rows
 * unwritten, it cannot cause an access outside the call's buffers.  plan == NULL is
 * acache_varlen_attn; head_dim other than 64 / 128 ignores the plan.  One plan serves every layer
 * of a forward pass (it depends on the lengths and head counts only).  No counterpart in the
 * reference, whose Triton grid is (query block, head, request) in launch order
 * (acache_attention.py:721-737).
 */
int acache_varlen_attn(
    void *out, const void *q, const void *k_cache, const void *v_cache,
    const int32_t *cu_q, const int32_t *cu_k, const int32_t *slot_map,
    float scale,
    int32_t shared_prefix_len, const int32_t *shared_kv_lens, const int32_t *affix_shifts,
    const float *rope_cos, const float *rope_sin, int32_t rope_rows,
    int32_t B, int64_t total_q, int64_t total_k,
    int32_t H, int32_t H_kv, int32_t D, int32_t dtype, int64_t num_slots,
    int64_t q_token_stride, int64_t q_head_stride,
    int64_t out_token_stride, int64_t out_head_stride,
    int64_t kv_slot_stride, int64_t kv_head_stride, void *stream);

int acache_varlen_attn_planned(
    void *out, const void *q, const void *k_cache, const void *v_cache,
    const int32_t *cu_q, const int32_t *cu_k, const int32_t *slot_map,
    float scale,
    int32_t shared_prefix_len, const int32_t *shared_kv_lens, const int32_t *affix_shifts,
    const float *rope_cos, const float *rope_sin, int32_t rope_rows,
    int32_t B, int64_t total_q, int64_t total_k,
    int32_t H, int32_t H_kv, int32_t D, int32_t dtype, int64_t num_slots,
    int64_t q_token_stride, int64_t q_head_stride,
    int64_t out_token_stride, int64_t out_head_stride,
    int64_t kv_slot_stride, int64_t kv_head_stride,
    const int32_t *plan, int64_t plan_blocks, void *stream);

/*
 * Host-side planner of acache_varlen_attn_planned: no GPU work, no device pointers.
 * cu_q_host / cu_k_host are HOST copies of the call's prefix sums (B + 1 entries each).
 * Returns the number of blocks of the plan (a multiple of 8, >= 0) or an ACACHE_E_* code.
 * With plan_host == NULL only the size is computed; otherwise 2 * blocks int32 are written
 * (capacity_blocks must be at least the returned size), to be copied to the device by the
 * caller.  Entry i is (request, tile | head << 20) for block i, request -1 = no work.
 * slots_per_xcd = workgroups of the attention kernel that one XCD holds at a time
 * (2 * CUs / 8; <= 0 selects 64, the MI355X value).  Every unit stays on the XCD that shares
 * its KV head's rows in L2; per XCD the units are packed into `slots_per_xcd` bins by a cost
 * model (a fixed part plus a term per 64-key tile, cheaper for tiles of at most 64 / 32 live
 * rows) and issued in the order of their start times in that packing.  Lists of at most one
 * unit per slot or of more than 16 per slot are issued longest first.  Host cost: about
 * 0.1 ms for a batch of 16 requests and 32 heads.
 */
int64_t acache_varlen_attn_plan(
    const int32_t *cu_q_host, const int32_t *cu_k_host, int32_t B, int32_t H, int32_t H_kv,
    int32_t slots_per_xcd, int32_t *plan_host, int64_t capacity_blocks);

/*
 * Two elementwise steps of the decoder block on either side of the attention path, for
 * hosts that run the model through this library (the package's own LLaDA / Dream mirror
 * does).  They sit outside the affix-reuse path proper; their reference counterparts are
 * model code: the SwiGLU of the MLP, act(ff_proj(x)) * up_proj(x), and the residual add in
 * front of the RMS layer norm (nano-vdllm/model/modeling_llada.py, block forward).
 *
 * acache_swiglu: out[t, j] = silu(gate_up[t, j]) * gate_up[t, m + j] for t < M, j < m, where a
 * row of gate_up holds the gate projection followed by the up projection (one merged GEMM).
 * silu in fp32, rounded to `dtype`, multiplied by the up value in fp32, rounded again (the
 * roundings of the separate activation and multiply kernels).  m * sizeof(dtype) must be a
 * multiple of 16; row strides in elements.
 *
 * acache_add_rms_norm: sum[t, :] = x[t, :] + delta[t, :] rounded to `dtype` (sum may be x itself;
 * with delta == NULL the sum is x and nothing is written to `sum`, which may then be NULL),
 * y[t, :] = round(sum[t, :] * rsqrt(mean(sum[t, :]^2) + eps)) * weight[:], statistics in fp32, the
 * normalised value rounded to `dtype` before the weight multiplies it (where the reference's RMS
 * layer norm rounds, llada/model/modeling_llada.py:338-350), the product rounded again.  y may not overlap the other rows.  d * sizeof(dtype) a multiple of 16 and at
 * most 16 KiB.
 */
int acache_swiglu(void *out, const void *gate_up, int64_t M, int64_t m,
                  int64_t in_row_stride, int64_t out_row_stride, int32_t dtype, void *stream);
int acache_add_rms_norm(void *sum, const void *x, const void *delta, const void *weight, void *y,
                        int64_t M, int64_t d, int64_t sum_row_stride, int64_t x_row_stride,
                        int64_t delta_row_stride, int64_t y_row_stride, float eps, int32_t dtype,
                        void *stream);

#ifdef __cplusplus
}
#endif
#endif /* ACACHE_HIP_H */
