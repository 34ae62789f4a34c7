/*
 * fp_paged_kv.h -- C ABI of libfp_paged_kv.so: the paged KV-cache path of
 * Falcon Perception as hand-written HIP kernels for gfx950 (MI355X).
 *
 * The reference implements this path in Python on top of torch
 * (falcon_perception/paged_attention.py, falcon_perception/attention.py); it has
 * no FFI of its own, so each entry point below names the reference function
 * whose device work it replaces.
 *
 * Conventions
 *  - Every pointer is a DEVICE pointer owned by the caller.  The library
 *    borrows it for the duration of the launch; it allocates and frees nothing.
 *  - `stream` is a hipStream_t passed as void*.  All work is enqueued on it and
 *    nothing synchronises, so the entry points may be captured in a HIP graph.  One
 *    condition: a kernel that keeps spilled registers in scratch memory must have been
 *    launched once on the device BEFORE a capture, because its first launch makes the
 *    runtime set that memory up, which it cannot do while a stream is being captured.
 *    The only such kernels here are those fp_paged_prefill launches at head_dim 64 for a
 *    launch that is not cut along the keys (bf16 and f16, 20 to 36 bytes per lane); every
 *    kernel behind the other entry points, and the rest of fp_paged_prefill, uses none
 *    (the build writes every kernel's figure to build/<source>.resources.txt and a test
 *    holds the list to exactly this).  The reference's engine captures decode steps only
 *    (paged_inference.py:916-935).
 *  - Strides are in ELEMENTS of the tensor's dtype, the innermost (head_dim)
 *    stride must be 1.
 *  - Return value: 0 on success, a negative FP_ERR_* code otherwise;
 *    fp_last_error() then holds a message for the calling thread.
 *  - Indices that fall outside the tables or the pool (a slot < 0 or >= n_slots,
 *    a batch index >= max_batch, a block id >= n_pages) are skipped on the
 *    device instead of faulting; the reference raises an index error there.
 *  - `n_pages` is the number of COLUMNS of page_table, i.e. the logical blocks one
 *    sequence can map.  The reference's table has one column per pool page
 *    (paged_attention.py:58); a narrower table [max_batch, max blocks per sequence]
 *    works the same and is what a pool of several hundred thousand pages needs.
 *    The pool's own page count is n_slots / page_size; page ids outside it count as
 *    unmapped.
 */
#ifndef FP_PAGED_KV_H
#define FP_PAGED_KV_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FP_ABI_VERSION 7

/* element types of pool / q / k / v */
#define FP_DTYPE_F32 0
#define FP_DTYPE_BF16 1
#define FP_DTYPE_F16 2

/* integer width of position / length arrays */
#define FP_INDEX_I32 0
#define FP_INDEX_I64 1

#define FP_OK 0
#define FP_ERR_INVALID_ARGUMENT (-1)
#define FP_ERR_UNSUPPORTED (-2)
#define FP_ERR_LAUNCH (-3)
#define FP_ERR_WORKSPACE (-4)

/* ABI version of the loaded library (FP_ABI_VERSION at build time). */
int fp_abi_version(void);

/* Message of the last failing call on this thread ("" if none). */
const char* fp_last_error(void);

/*
 * KV append: slot-mapping scatter of new K/V rows into the page pool.
 * Replaces PagedKVCache.assign (paged_attention.py:184-232; clamp_negative = 1:
 * stale -1 table entries go to page 0, :222) and
 * PagedKVCache.assign_prefill_no_paging (paged_attention.py:364-393;
 * clamp_negative = 0: a negative slot wraps from the end of the slot axis as the
 * reference's negative index does, :389-391).
 *
 *   pool_k, pool_v   [H, n_slots, D]   one layer's K and V planes of kv_cache
 *   k, v             [T, H, S, D] with element strides (t, h, s); bytes are copied
 *                    unchanged.  Prefill [1, H, L, D] is passed as T = L, S = 1,
 *                    stride_t = the stride of the L axis.
 *   page_table       [max_batch, n_pages] int64, row stride pt_row_stride
 *   batch_idx        [T] int64  cache slot of each row group
 *   input_pos        [T, S] contiguous, int32 or int64 (pos_index_type)
 * Row (t, s) of head h goes to
 *   pool[h, page_table[batch_idx[t], pos / page_size] * page_size + pos % page_size, :].
 */
int fp_kv_append(void* pool_k, void* pool_v,
                 const void* k, const void* v,
                 int64_t k_stride_t, int64_t k_stride_h, int64_t k_stride_s,
                 int64_t v_stride_t, int64_t v_stride_h, int64_t v_stride_s,
                 const int64_t* page_table, int64_t pt_row_stride,
                 const int64_t* batch_idx,
                 const void* input_pos, int pos_index_type,
                 int32_t T, int32_t H, int32_t S, int32_t D,
                 int32_t page_size, int32_t n_pages, int32_t max_batch,
                 int64_t n_slots, int dtype, int clamp_negative,
                 void* stream);

/*
 * Page gather: the logical view of cached sequences, the inverse of fp_kv_append.
 * The reference gathers pages implicitly inside its attention kernels through the
 * converted block indices (paged_attention.py:279-284); this is that lookup as a
 * standalone bit copy.
 *
 *   pool   [H, n_slots, D]
 *   out    [B, H, max_len, D] with element strides (b, h, t)
 *   out[b, h, t, :] = pool[h, page_table[batch_idx[b], t / P] * P + t % P, :]
 *                     for t < seq_lens[b], zero for seq_lens[b] <= t < max_len.
 */
int fp_kv_gather(const void* pool, void* out,
                 int64_t out_stride_b, int64_t out_stride_h, int64_t out_stride_t,
                 const int64_t* page_table, int64_t pt_row_stride,
                 const int64_t* batch_idx,
                 const void* seq_lens, int len_index_type,
                 int32_t B, int32_t H, int32_t max_len, int32_t D,
                 int32_t page_size, int32_t n_pages, int32_t max_batch,
                 int64_t n_slots, int dtype,
                 void* stream);

/*
 * Logical -> physical block ids of a block mask.
 * Replaces the zeros + torch.gather pair in
 * PagedKVCache.convert_logical_block_mask (paged_attention.py:279-284).
 *
 *   kv_indices   [B, rows_per_batch, C] int32 contiguous (rows_per_batch = H*ROWS)
 *   out          [B, rows_per_batch, n_pages] int32 contiguous
 *   out[b, r, c] = (int32) page_table[batch_idx[b], kv_indices[b, r, c]] for c < C, else 0.
 */
int fp_convert_block_ids(const int32_t* kv_indices, int32_t* out,
                         const int64_t* page_table, int64_t pt_row_stride,
                         const int64_t* batch_idx,
                         int32_t B, int32_t rows_per_batch, int32_t C,
                         int32_t n_pages, int32_t max_batch,
                         void* stream);

/*
 * Split size (tokens per split-K partition) fp_paged_decode picks when called with
 * split_tokens = 0 for this shape; use it to size the workspace.
 */
int32_t fp_paged_decode_default_split(int32_t B, int32_t Hc, int32_t max_context, int32_t page_size);

/*
 * Bytes of workspace fp_paged_decode needs for the given launch shape
 * (split-K partial results: B * Hq * ceil(max_context / split_tokens) * (D + 2) floats;
 * nothing when one split covers max_context).  max_context bounds input_pos + 1,
 * split_tokens is an explicit multiple of 64.
 * Returns a negative FP_ERR_* code for a bad argument.
 */
int64_t fp_paged_decode_workspace_bytes(int32_t B, int32_t Hq, int32_t D,
                                        int32_t max_context, int32_t split_tokens);

/*
 * Split-K paged decode attention (one query token per sequence) + cross-split merge.
 * Replaces compiled_flex_attn_decode (attention.py:17) as called at
 * model.py:156-162 on the pool views returned by PagedKVCache.assign, together
 * with the per-step mask plumbing it depends on (paged_inference.py:783-826,
 * paged_attention.py:234-333): pages are looked up in page_table directly.
 *
 *   q        [B, Hq, 1, D], element strides (b, h)
 *   pool_k/v [Hc, n_slots, D], Hq % Hc == 0; query head h reads cache head h / (Hq/Hc)
 *   input_pos[B] int32/int64: sequence b attends logical positions 0..input_pos[b]
 *   out      [B, Hq, 1, D] same dtype as q, element strides (b, h)
 *   lse      [B, Hq] float32, natural log of the softmax denominator
 *   kv_rep   1, or (2, 4) for a cache that stores one head per query head (Hc = Hq) whose V heads
 *            are kv_rep identical copies while the K heads differ -- what the reference's
 *            repeat_kv before the per-head rotary embedding produces (model.py:112-114).  The
 *            kernel then reads the kv_rep K rows of a group and one V row (the first copy)
 *            instead of kv_rep of each; results equal those of kv_rep = 1 on such a cache
 *   sinks    NULL, or [Hq] float32: out is multiplied by sigmoid(lse - sinks[h]), the
 *            attention-sink gate of Attention._post_attention (model.py:122-128), with the
 *            reference's rounding (attention output rounded to the dtype, product rounded again);
 *            lse is returned ungated.  With strides (Hq * D, D) out is then the [B, 1, Hq * D]
 *            row the reference's output projection takes (model.py:127-128)
 *   scale    multiplies q.k (1/sqrt(D) in the reference)
 *   max_context   upper bound of input_pos + 1, fixes the launch grid
 *   split_tokens  tokens per split, a multiple of 64 (0 = library default)
 *   plan     NULL, or the plan fp_paged_decode_plan wrote for THIS step and launch shape (plan_bytes >=
 *            fp_paged_decode_plan_bytes()).  Results are bit-identical with and without it.
 * A sequence with input_pos < 0 yields out = 0, lse = -inf.
 */
int64_t fp_paged_decode_plan_bytes(void);

/*
 * The plan of a decode step.  The reference converts its block mask once per step
 * (paged_inference.py:847-848) and every layer's attention consumes it (model.py:689-699); here the
 * corresponding per-step work is what a workgroup of a large launch (the even cut) has to find out
 * before it can ask for its first K row: which sequences its chunk covers, their lengths and the page
 * ids of its rows (positions -> cut -> page table, dependent loads in every workgroup of every layer).
 * fp_paged_decode_plan does that once, into `plan`; the decode entry points of the same step and the same
 * shape (B, Hq, Hc, kv_rep, D, page_size, max_context, split_tokens, dtype) then start from one load.
 * Takes the arguments of the decode call it serves; q, pool_k, pool_v, out, lse and workspace are not
 * touched and may be NULL.  Between this call and the launches that use the plan, input_pos, batch_idx and the
 * rows of page_table they name must not change.  A workgroup that finds a plan made for another B or
 * max_context ignores it.  A plan of the right shape made from other positions or slots is found out by
 * the merge pass (it reads both anyway and compares a hash of them with the plan's): out and lse are then
 * NaN in every row, and a fused append has stored the fresh rows of the sequences that moved where the plan
 * said; changed rows of the page table are not detected.  A launch that goes split by split (a few
 * sequences) has no use for a plan: the call then launches nothing and the buffer is ignored.
 * No counterpart in the reference's kernels; capturable like every other entry point.
 */
int fp_paged_decode_plan(const void* q, int64_t q_stride_b, int64_t q_stride_h,
                         const void* pool_k, const void* pool_v,
                         const int64_t* page_table, int64_t pt_row_stride,
                         const int64_t* batch_idx,
                         const void* input_pos, int pos_index_type,
                         void* out, int64_t out_stride_b, int64_t out_stride_h,
                         float* lse, const float* sinks,
                         void* workspace, int64_t workspace_bytes,
                         int32_t B, int32_t Hq, int32_t Hc, int32_t kv_rep, int32_t D,
                         int32_t page_size, int32_t n_pages, int32_t max_batch,
                         int64_t n_slots, int32_t max_context, int32_t split_tokens,
                         float scale, int dtype,
                         void* plan, int64_t plan_bytes,
                         void* stream);

int fp_paged_decode(const void* q, int64_t q_stride_b, int64_t q_stride_h,
                    const void* pool_k, const void* pool_v,
                    const int64_t* page_table, int64_t pt_row_stride,
                    const int64_t* batch_idx,
                    const void* input_pos, int pos_index_type,
                    void* out, int64_t out_stride_b, int64_t out_stride_h,
                    float* lse, const float* sinks,
                    void* workspace, int64_t workspace_bytes,
                    int32_t B, int32_t Hq, int32_t Hc, int32_t kv_rep, int32_t D,
                    int32_t page_size, int32_t n_pages, int32_t max_batch,
                    int64_t n_slots, int32_t max_context, int32_t split_tokens,
                    float scale, int dtype,
                    void* plan, int64_t plan_bytes,
                    void* stream);

/*
 * The two passes of fp_paged_decode as separate calls, same arguments: the partial pass
 * leaves, per (sequence, query head, piece of the context), the unnormalised accumulator,
 * running maximum and denominator in the workspace (log2 units); the merge pass combines
 * them into out and lse.  The pieces are the splits of split_tokens tokens
 * ([B, Hq, n_splits, D] floats followed by [B, Hq, n_splits, 2] floats), except that a
 * launch of more workgroups than the GPU holds at once is cut into equal chunks of the
 * contexts laid end to end (rows (chunk + sequence) * Hq + head of [rows, D] and [rows, 2]
 * floats): the layout is a matter between the two passes.  For callers that time or
 * overlap the passes.  No counterpart in the
 * reference, whose Triton decode kernel keeps both passes internal
 * (torch/_inductor/kernel/flex/flex_decoding.py:229).  When one split covers
 * max_context the partial pass writes out and lse itself and the merge pass does nothing.
 */
int fp_paged_decode_partial(const void* q, int64_t q_stride_b, int64_t q_stride_h,
                            const void* pool_k, const void* pool_v,
                            const int64_t* page_table, int64_t pt_row_stride,
                            const int64_t* batch_idx,
                            const void* input_pos, int pos_index_type,
                            void* out, int64_t out_stride_b, int64_t out_stride_h,
                            float* lse, const float* sinks,
                            void* workspace, int64_t workspace_bytes,
                            int32_t B, int32_t Hq, int32_t Hc, int32_t kv_rep, int32_t D,
                            int32_t page_size, int32_t n_pages, int32_t max_batch,
                            int64_t n_slots, int32_t max_context, int32_t split_tokens,
                            float scale, int dtype,
                            void* plan, int64_t plan_bytes,
                            void* stream);
int fp_paged_decode_merge(const void* q, int64_t q_stride_b, int64_t q_stride_h,
                          const void* pool_k, const void* pool_v,
                          const int64_t* page_table, int64_t pt_row_stride,
                          const int64_t* batch_idx,
                          const void* input_pos, int pos_index_type,
                          void* out, int64_t out_stride_b, int64_t out_stride_h,
                          float* lse, const float* sinks,
                          void* workspace, int64_t workspace_bytes,
                          int32_t B, int32_t Hq, int32_t Hc, int32_t kv_rep, int32_t D,
                          int32_t page_size, int32_t n_pages, int32_t max_batch,
                          int64_t n_slots, int32_t max_context, int32_t split_tokens,
                          float scale, int dtype,
                          void* plan, int64_t plan_bytes,
                          void* stream);

/*
 * Decode step in one call: append the newest K/V row of every sequence AND attend over the
 * context including it.  Equivalent to fp_kv_append(clamp_negative = 1, S = 1) at position
 * input_pos[b] followed by fp_paged_decode, i.e. to PagedKVCache.assign
 * (paged_attention.py:184-232) + compiled_flex_attn_decode (model.py:150-162), without the
 * separate append launch: the workgroup that owns position input_pos[b] takes that row from
 * k_new / v_new, folds it into the attention and writes it to its pool slot.
 *
 *   k_new, v_new  [B, Hc, 1, D], element strides (b, h); pool_k / pool_v are written
 * A sequence with input_pos >= max_context lies outside what the launch was sized for: its fresh row
 * is neither stored nor attended, the pool stays as it was, and the result covers positions
 * 0 .. max_context - 1 as fp_paged_decode would return it.
 * All other arguments as fp_paged_decode.
 */
int fp_paged_decode_append(const void* k_new, const void* v_new,
                           int64_t k_stride_b, int64_t k_stride_h,
                           int64_t v_stride_b, int64_t v_stride_h,
                           const void* q, int64_t q_stride_b, int64_t q_stride_h,
                           const void* pool_k, const void* pool_v,
                           const int64_t* page_table, int64_t pt_row_stride,
                           const int64_t* batch_idx,
                           const void* input_pos, int pos_index_type,
                           void* out, int64_t out_stride_b, int64_t out_stride_h,
                           float* lse, const float* sinks,
                           void* workspace, int64_t workspace_bytes,
                           int32_t B, int32_t Hq, int32_t Hc, int32_t kv_rep, int32_t D,
                           int32_t page_size, int32_t n_pages, int32_t max_batch,
                           int64_t n_slots, int32_t max_context, int32_t split_tokens,
                           float scale, int dtype,
                           void* plan, int64_t plan_bytes,
                           void* stream);

/*
 * fp_paged_decode without a workspace argument, for callers that cannot allocate device memory:
 * code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  No counterpart
 * in the reference.  The split-K partial results go to an array of FP_NOALLOC_SCRATCH_BYTES that is
 * part of the library's device image (every GPU the library runs on holds its own copy until the
 * process ends); the call allocates and frees nothing.  The first call on a device looks the array's
 * address up once (hipGetSymbolAddress, with that device current), which may make the runtime load the
 * library's device image: make that first call OUTSIDE a graph capture (any small launch will do);
 * every later call on the device may be captured.
 *  - A launch whose partial results (fp_paged_decode_workspace_bytes for the same shape) exceed
 *    FP_NOALLOC_SCRATCH_BYTES is refused with FP_ERR_WORKSPACE.
 *  - All calls on one GPU share that GPU's array: calls that overlap there (different streams or
 *    threads) race.  Nothing needs clearing between calls.
 * Arguments and results as fp_paged_decode.
 */
#define FP_NOALLOC_SCRATCH_BYTES (64ll << 20)
int fp_paged_decode_noalloc(const void* q, int64_t q_stride_b, int64_t q_stride_h,
                            const void* pool_k, const void* pool_v,
                            const int64_t* page_table, int64_t pt_row_stride,
                            const int64_t* batch_idx,
                            const void* input_pos, int pos_index_type,
                            void* out, int64_t out_stride_b, int64_t out_stride_h,
                            float* lse, const float* sinks,
                            int32_t B, int32_t Hq, int32_t Hc, int32_t kv_rep, int32_t D,
                            int32_t page_size, int32_t n_pages, int32_t max_batch,
                            int64_t n_slots, int32_t max_context, int32_t split_tokens,
                            float scale, int dtype,
                            void* stream);

/*
 * Tail of Attention._pre_attention (model.py:110-119) and the cache insert that follows it
 * (model.py:150-153 -> PagedKVCache.assign / assign_prefill_no_paging, paged_attention.py:184-232,
 * 364-393) in one pass: RMS norm of q and k over head_dim (no weight), repeat of k and v to the
 * cached head count, 3D rotary embedding (rope.py:88-108: 1D on the first half of head_dim with
 * freqs_cis, "golden" 2D on the second half with per-head freqs_cis_2d when given), rotated q
 * written in the caller's layout, K and V rows written to their pool slots.  Removes the
 * repeat_kv / permute / .contiguous() copies and the separate append launch.
 *
 *   xq [T, Hq, D], xk, xv [T, Hkv, D] views with element strides (token, head): the slices of the
 *              qkv projection, T = all tokens of the step (B for decode, packed length for prefill)
 *   freqs_cis     [T, D/4, 2] float32 (cos, sin) = view_as_real of the reference's complex64 [.., D/4]
 *   freqs_cis_2d  NULL or [T, Hq, D/4, 2] float32; needs H_pool == Hq
 *   q_out      [T, Hq, D] view, element strides (token, head), e.g. those of a [B, H, S, D] tensor
 *   pool_k/v   [H_pool, n_slots, D]; cached head h takes source head h / (H_pool / Hkv)
 *   batch_idx, input_pos [T]: cache slot and position of every token
 *   eps        added to mean(x^2); the reference passes eps=None, for which torch takes 2^-23
 *              (the epsilon of the fp32 computation type) for every dtype
 *   clamp_negative  as fp_kv_append (1 = decode semantics, 0 = prefill semantics)
 * Rounding follows the reference: norm result rounded to dtype, rotation in fp32, rounded again.
 */
int fp_qkv_norm_rope_append(const void* xq, const void* xk, const void* xv,
                            int64_t q_stride_t, int64_t q_stride_h,
                            int64_t k_stride_t, int64_t k_stride_h,
                            int64_t v_stride_t, int64_t v_stride_h,
                            const float* freqs_cis, const float* freqs_cis_2d,
                            void* q_out, int64_t qo_stride_t, int64_t qo_stride_h,
                            void* pool_k, void* pool_v,
                            const int64_t* page_table, int64_t pt_row_stride,
                            const int64_t* batch_idx,
                            const void* input_pos, int pos_index_type,
                            int32_t T, int32_t Hq, int32_t Hkv, int32_t H_pool, int32_t D,
                            int32_t page_size, int32_t n_pages, int32_t max_batch,
                            int64_t n_slots, float eps, int dtype, int clamp_negative,
                            void* stream);

/*
 * Per-row key limits of the hybrid mask (bidirectional inside an image span,
 * causal elsewhere).  Replaces the compiled create_block_mask evaluation of
 * create_prefill_blockmask (paged_attention.py:343-362) with
 * get_image_prefix_mask_mod (attention.py:75-96) by a closed form.
 *
 *   input_ids [L] int64 packed token ids, soi_id / eoi_id the span delimiters
 *   batch_idx NULL, or [L] int64 cache slot of each packed row (the documents of the row); needed
 *             for status bit 1 and for open_at_start
 *   open_at_start  NULL, or [max_batch] bytes: slot s != 0 declares that the first row of slot s in
 *             this packed row lies inside an image span whose soi was prefilled by an earlier chunk
 *             (no counterpart in the reference, whose engine prefills whole sequences,
 *             paged_inference.py:637-672); the rows up to the span's eoi then get the eoi's index
 *   row_hi    [L] int32 out: packed index one past the last key row q may see
 *             = max(q + 1, end of q's image span)
 *   status    NULL, or one int32 out (written, not accumulated): 0 when row_hi is the mask of a packed
 *             row of whole sequences.  Delimiters are counted over the WHOLE packed row, as the
 *             reference's mask counts them (attention.py:77-79), not per document:
 *             bit 0 = at some token more eoi than soi (virtual ones included) have been seen: an eoi
 *             with no span open.  row_hi is then still what the reference's predicate gives for this
 *             row (nothing is inside a span while the balance is not positive), which is the right
 *             mask for a stray eoi and the wrong one for a chunk that starts inside a span and was
 *             not declared;
 *             bit 1 = the balance is positive where batch_idx changes or the row ends: a span still
 *             open there (its rows would need keys of another document or keys not yet cached).
 *             row_hi is then not a usable mask and the caller must reject the step.  An eoi of the
 *             NEXT document closes such a span in the global count, so bit 0 is not raised with it.
 * L <= 65536 (one workgroup scans the row).
 */
int fp_hybrid_row_limits(const int64_t* input_ids, const int64_t* batch_idx,
                         const uint8_t* open_at_start, int32_t max_batch, int32_t L,
                         int64_t soi_id, int64_t eoi_id,
                         int32_t* row_hi, int32_t* status, void* stream);

/*
 * Chunked-prefill attention over the paged cache under the hybrid mask, on the matrix
 * instructions of the dtype (bf16, f16, fp32).
 * Replaces compiled_flex_attn_prefill (attention.py:18) as called at model.py:156-162,
 * extended to read the prefix from pages (the reference attends over the packed
 * fresh K/V only, paged_attention.py:393).
 *
 *   q          [Lq, Hq, D] view with element strides (row, head) of the packed rows
 *   batch_idx  [Lq] int64 cache slot of each row (0 = padding: out 0, lse -inf)
 *   row_limit  [Lq] int32 logical keys 0..row_limit-1 of the row's sequence are visible
 *              (row position + 1 for a causal row, the end of the image span inside one);
 *              every such key must already be in the pages
 *   out        [Lq, Hq, D] view, strides (row, head); lse [Hq, Lq] float32
 *   sinks      NULL, or [Hq] float32 attention-sink logits, as in fp_paged_decode
 *   score_bound  0 when nothing is known about the scores; otherwise the caller's guarantee that
 *              |scale * q.k| <= score_bound for every visible (query, key) pair of the launch.  The
 *              reference's model RMS-normalises q and k without a weight and rotates them
 *              (model.py:110-116), so |q| = |k| = sqrt(D) and score_bound = sqrt(D) holds by
 *              construction.  With 0 < score_bound <= 40 the bf16 kernel drops the running maximum of
 *              the online softmax: Q is multiplied by scale * log2(e) when it is loaded (and rounded to
 *              bf16 again), and the probabilities are exp2 of the matrix product itself, referred to the
 *              fixed point 0.  Results agree with the unbounded path within bf16 rounding.  A bound
 *              the data breaks gives wrong results only once exp2(score * log2 e) leaves fp32's
 *              range.  f16 and fp32 ignore the argument.
 *   workspace  NULL, or workspace_bytes bytes of device memory, 16-byte aligned (no need to clear it).
 *              A launch with fewer workgroups than the GPU needs (few query rows, few heads) is then
 *              also cut along the keys: up to 8 workgroups share a query tile, each takes an equal part
 *              of the keys, and a merge pass combines them (two launches instead of one).  Without a
 *              workspace, or with one that is too small, the cut is coarser or absent; results agree
 *              within rounding.
 */
/* Bytes of workspace with which fp_paged_prefill cuts a launch of this shape as finely as it would like
 * to on the current device (0: it would not cut it at all); a negative FP_ERR_* for a bad argument. */
int64_t fp_paged_prefill_workspace_bytes(int32_t Lq, int32_t Hq, int32_t Hc, int32_t D, int dtype);

/*
 * The order of a prefill launch's workgroups (optional; no counterpart in the reference).  The GPU hands the
 * workgroups of a launch out in the order of their ids, and a launch ends with its last workgroup: the ids should
 * run from the query tile with the longest key range to the one with the shortest.  By itself fp_paged_prefill
 * takes the tiles by descending row index, which is that order inside one sequence but not across a packed row of
 * several.  fp_paged_prefill_tile_order writes the exact order for a step - once per step, from the step's
 * batch_idx and row_limit; every layer's fp_paged_prefill takes it as `tile_order` - and pays where several
 * small workgroups share a CU (head_dim 64: 8 x 512-row chunks 65 us against 73 us, whole sequences 266 us
 * against 278 us); at head_dim 128 it changes nothing.  The ranking itself takes 5 us at 4096 rows, 21 us at 23040.  Results are bit-identical with and without.
 *   fp_paged_prefill_tile_rows   rows per query tile of the launch fp_paged_prefill makes for this shape and
 *                                workspace size (32 .. 256; 0: the launch takes no order - fp32)
 *   fp_paged_prefill_tile_order  order[ceil(Lq / tile_rows)] int32: query tiles by decreasing key range (the
 *                                largest row_limit of the tile's rows, padding rows counting as 0); at most
 *                                4096 tiles
 * fp_paged_prefill uses `tile_order` only if `tile_order_rows` is the tile size of its launch, NULL / 0: none.
 */
int32_t fp_paged_prefill_tile_rows(int32_t Lq, int32_t Hq, int32_t Hc, int32_t D, int dtype, int64_t workspace_bytes);
int fp_paged_prefill_tile_order(const int64_t* batch_idx, const int32_t* row_limit, int32_t Lq, int32_t tile_rows,
                                int32_t* order, void* stream);

int fp_paged_prefill(const void* q, int64_t q_stride_row, int64_t q_stride_h,
                     const void* pool_k, const void* pool_v,
                     const int64_t* page_table, int64_t pt_row_stride,
                     const int64_t* batch_idx, const int32_t* row_limit,
                     void* out, int64_t out_stride_row, int64_t out_stride_h,
                     float* lse, const float* sinks,
                     int32_t Lq, int32_t Hq, int32_t Hc, int32_t D,
                     int32_t page_size, int32_t n_pages, int32_t max_batch,
                     int64_t n_slots, float scale, float score_bound, int dtype,
                     void* workspace, int64_t workspace_bytes,
                     const int32_t* tile_order, int32_t tile_order_rows,
                     void* stream);

/*
 * A measuring kernel, not an operator (no counterpart in the reference; nothing of the attention path calls it):
 * every wavefront runs 2 * iters times what one wavefront of the bf16 prefill kernel does per 64-key tile at
 * head_dim 128 with a score bound - 32 v_mfma_f32_32x32x16_bf16 with their K and V operands read from LDS
 * (mode 0), the softmax of 32 scores per lane: 32 exp2, 32 additions, 16 packs to bf16 (mode 1), or both in
 * turn (mode 2) - and nothing else: no staging, barrier, mask or address arithmetic.  `workgroups` workgroups of
 * 256 * waves_per_simd threads (waves_per_simd 1 .. 3; one workgroup fits a CU); `out` takes one float per
 * launched thread.  Timed by the caller (bench.py --overlap-probe): what it shows is how much of the vector
 * work a SIMD hides behind the matrix work of another wavefront, which bounds what the prefill kernel's
 * schedule can reach.
 */
int fp_probe_mfma_softmax(int mode, int waves_per_simd, int workgroups, int iters, float* out, int64_t out_floats,
                          void* stream);

#ifdef __cplusplus
}
#endif
#endif /* FP_PAGED_KV_H */
