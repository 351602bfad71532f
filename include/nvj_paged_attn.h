/*
 * C ABI of the MI355X (gfx950) paged-decode path: KV-cache store and split-K
 * paged decode attention.
 *
 * Every entry point takes plain device pointers, sizes and a HIP stream
 * (passed as void* so the header needs no HIP include), only ENQUEUES work on
 * that stream, never synchronises, never allocates and is re-entrant: the
 * library keeps no state between calls other than two per-device look-ups it
 * makes once (the number of compute units, the address of the array behind
 * nvj_paged_decode_static_launch) and that array itself.  Return value: 0 on
 * success, a negative NVJ_ERR_* code otherwise (never throws, never exits); the
 * code reflects this call only (a launch reports its own status and does not
 * read or clear the calling thread's HIP last-error slot).  Data pointers
 * (q, out, caches, K/V rows, workspace, activations) must be 16-byte aligned,
 * int32 metadata 4-byte aligned: NVJ_ERR_ALIGNMENT otherwise, from every entry
 * point.  Citations name the reference interface each entry point stands in
 * for (paths relative to the reference checkout).
 */
#ifndef NVJ_PAGED_ATTN_H_
#define NVJ_PAGED_ATTN_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define NVJ_ABI_VERSION 3

/* exported from the shared library (which is built with hidden visibility) */
#define NVJ_API __attribute__((visibility("default")))

/* error codes */
#define NVJ_OK                 0
#define NVJ_ERR_NULL_POINTER  -1   /* a required pointer is NULL                    */
#define NVJ_ERR_BAD_SHAPE     -2   /* negative size, Hq % Hkv != 0, ...             */
#define NVJ_ERR_UNSUPPORTED   -3   /* head_dim / group size / block size not built  */
#define NVJ_ERR_WORKSPACE     -4   /* workspace missing or too small                */
#define NVJ_ERR_LAUNCH        -5   /* the kernel launch itself reported an error     */
#define NVJ_ERR_BAD_DTYPE     -6   /* unknown element type code                     */
#define NVJ_ERR_SCRATCH_LIMIT -7   /* nvj_paged_decode_static_launch: the problem needs
                                      more than NVJ_STATIC_SCRATCH_BYTES of scratch  */
#define NVJ_ERR_ALIGNMENT     -8   /* a data pointer is not 16-byte aligned (every
                                      entry point; int32 metadata needs 4 bytes)    */

#define NVJ_CHUNK_WHOLE_SEQUENCE (-1)   /* see the split modes of the paged decode */

/* element type codes: the cache (and q / out) is bf16 or IEEE half; float32 is
 * accepted only for the new K/V rows handed to the store */
#define NVJ_DTYPE_BF16 0
#define NVJ_DTYPE_F32  1
#define NVJ_DTYPE_F16  2

/* Human-readable text for an NVJ_ERR_* code (static storage). */
NVJ_API const char* nvj_error_string(int code);

/* NVJ_ABI_VERSION the library was built with. */
NVJ_API int nvj_abi_version(void);

/*
 * KV-cache store.  Replaces store_kv_to_cache (layers/attention.py:42-77) as
 * called from Attention.__call__ on the flattened cache
 * (layers/attention.py:457-475).
 *
 *   key   [num_tokens, num_kv_heads, head_dim]  k_dtype: cache_dtype, or f32 (the
 *         reference hands over f32 keys after RoPE and casts, :70)
 *   value [num_tokens, num_kv_heads, head_dim]  v_dtype: cache_dtype or f32
 *   k_cache, v_cache [num_slots, num_kv_heads, head_dim] cache_dtype (bf16 or
 *         f16, the model dtype of the reference, engine/model_runner.py:176),
 *         updated IN PLACE (num_slots = num_blocks * block_size)
 *   slot_mapping [num_tokens] int32
 *
 * cache[slot[i]] = round_nearest_even_to_cache_dtype(x[i]) for 0 <= slot[i] < num_slots;
 * slot[i] >= num_slots is dropped (mode='drop', :74); slot[i] < 0 is SKIPPED
 * (the documented meaning of -1, :57-58 -- the reference's code would write
 * row 0 instead).  Rows not named by slot_mapping are not touched.  Duplicate
 * slots: one of the writers wins, unspecified which (as in the reference).
 * num_tokens == 0 is a no-op.  head_dim * num_kv_heads must be a multiple of 8.
 */
NVJ_API int nvj_store_kvcache_launch(void* stream,
                             const void* key, const void* value,
                             void* k_cache, void* v_cache,
                             const int32_t* slot_mapping,
                             int32_t num_tokens, int32_t num_kv_heads,
                             int32_t head_dim, int64_t num_slots,
                             int32_t k_dtype, int32_t v_dtype, int32_t cache_dtype);

/*
 * How the positions of a call are split over workgroups is chosen by `chunk`:
 *
 *   chunk == 0  balanced split (the default), ONE launch for any mix of
 *               lengths, at most one 8-wave workgroup per CU.  The kernel reads
 *               context_lens on the device and lays the work out itself, so
 *               ragged batches are balanced without the host knowing the
 *               lengths.  Where whole (sequence, head group) rows can be dealt
 *               to the workgroups within a quarter of an equal share of the
 *               32-position steps (lengths equal or nearly so; or, taken by
 *               decreasing length, long rows that pair up with short ones,
 *               if need be with rows of half as many KV heads), no row is
 *               shared between workgroups and the workspace is not touched (the launch is bound by the memory system as a whole,
 *               so an uneven deal costs far less than its unevenness, and
 *               less than sharing rows does).  Otherwise the steps of all rows, end to end, are cut
 *               into equal runs, one per wave; a row that fits one workgroup is
 *               finished there, a row shared by several is merged by the wave
 *               that completes it (counters in the workspace), without a
 *               second launch.
 *   chunk  > 0  fixed split: workgroup (b, c) takes positions
 *               [c * chunk, (c + 1) * chunk) of sequence b; chunk must be a
 *               multiple of 32.
 *   chunk == NVJ_CHUNK_WHOLE_SEQUENCE (-1)
 *               every sequence is finished inside one workgroup: a workgroup
 *               owns 1, 2, 4 or 8 KV heads of one sequence (as many as still
 *               give 256 workgroups) and its 8 waves split the sequence's
 *               positions between them, merging through LDS.  No workspace, no
 *               second pass.  For the caller that knows (as the reference's
 *               host filler does, engine/model_runner.py:334-376) that the
 *               sequences of the batch have similar lengths and that
 *               batch * num_kv_heads is large enough to fill the GPU; a ragged
 *               batch is better served by chunk == 0.
 *
 * nvj_paged_decode_default_chunk: the fixed chunk the library recommends for a
 * problem of this shape when a fixed split is wanted (a multiple of 32).
 */
NVJ_API int32_t nvj_paged_decode_default_chunk(int32_t batch, int32_t num_kv_heads,
                                       int32_t max_blocks, int32_t block_size);

/*
 * Number of workgroups chunk == NVJ_CHUNK_WHOLE_SEQUENCE launches for a batch:
 * batch * num_kv_heads / (KV heads per workgroup; a cache head with more than
 * 16 query heads counts as several).  One 8-wave workgroup is
 * resident per CU (256 on MI355X), so that mode pays off when this is (just
 * under) a multiple of 256 and the lengths are similar; 0 on invalid arguments.
 */
NVJ_API int32_t nvj_paged_decode_whole_sequence_workgroups(int32_t batch, int32_t num_heads,
                                                   int32_t num_kv_heads);

/*
 * Bytes of device workspace nvj_paged_decode_launch needs for the given `chunk`
 * mode: the partials (fp32 accumulators plus running max and sum per partial)
 * and, in balanced mode, in front of them one int32 counter per (sequence, KV
 * head).  Returns 0 on invalid arguments, and for chunk ==
 * NVJ_CHUNK_WHOLE_SEQUENCE, which needs none (workspace may then be NULL).  The
 * balanced size depends on the number of compute units of the current device.
 *
 * nvj_paged_decode_counter_bytes: how many bytes at the head of a balanced-split
 * workspace are its counter region (int32 words: word 0 is the stale flag
 * described at nvj_paged_decode_launch_phases, then one counter per (sequence,
 * KV head); padded to 256 bytes; 0 on invalid arguments).  What lies behind it
 * holds partials; nvj_paged_decode_launch_counters takes the two as separate
 * buffers.
 */
NVJ_API size_t nvj_paged_decode_counter_bytes(int32_t batch, int32_t num_heads,
                                             int32_t num_kv_heads);

NVJ_API size_t nvj_paged_decode_workspace_bytes(int32_t batch, int32_t num_heads,
                                        int32_t head_dim, int32_t max_blocks,
                                        int32_t block_size, int32_t num_kv_heads,
                                        int32_t chunk);

/*
 * Paged decode attention, one query position per sequence.  Replaces
 * paged_attention (layers/pallas_attention.py:465-507) ->
 * paged_decode_attention_vectorized (:146-238) as dispatched from
 * Attention._decode_attention (layers/attention.py:389-397), and equally the
 * gather + dot_product_attention fallback (layers/attention.py:399-434).
 *
 *   q            [batch, num_heads, head_dim]                         dtype
 *   k_cache, v_cache [num_blocks, block_size, num_kv_heads, head_dim] dtype
 *   block_tables [batch, max_blocks] int32; entries at or beyond
 *                ceil(context_lens[b] / block_size) are never read (the
 *                reference pads them with -1, engine/model_runner.py:240)
 *   context_lens [batch] int32 (counts the position being decoded,
 *                engine/model_runner.py:360)
 *   out          [batch, num_heads, head_dim]                         dtype
 *   workspace    >= nvj_paged_decode_workspace_bytes(...) bytes, 16-byte aligned,
 *                contents need not be initialised (this entry point clears the
 *                counters of the balanced split itself, with a small kernel
 *                ahead of the main one)
 *
 * out[b,h,:] = softmax_{s < ctx[b]}(scale * q[b,h,:] . K[b,s,h/G,:]) V[b,s,h/G,:]
 * with G = num_heads / num_kv_heads, fp32 accumulation, result in `dtype`
 * (NVJ_DTYPE_BF16 or NVJ_DTYPE_F16: the cache dtype of the reference is its model
 * dtype, and its own timing scripts use float16).
 * context_lens[b] <= 0 gives a row of zeros (0 / (0 + 1e-9), :227).  Positions
 * >= context_lens[b] are never read.  Table entries of live pages must lie in
 * [0, num_blocks); the kernel clamps them into range like the reference (:185)
 * rather than faulting.
 *
 * Launches on `stream`: chunk == 0: the counter-clearing kernel and the
 * attention kernel; chunk > 0: the split-K kernel and the combine pass; chunk
 * == NVJ_CHUNK_WHOLE_SEQUENCE: one kernel.
 * Supported: head_dim 128 (every Qwen3 size) or 64 (the reference's toy test
 * shapes), block_size a multiple of 32, chunk a multiple of 32 (0 = balanced
 * split) or NVJ_CHUNK_WHOLE_SEQUENCE.  K/V are read once for up to 16 query
 * heads per KV head (every Qwen3 size has 2 to 8); a larger group is served in
 * parts of at most 16, with one read of the KV head's rows per part.
 */
NVJ_API int nvj_paged_decode_launch(void* stream,
                            const void* q, const void* k_cache, const void* v_cache,
                            const int32_t* block_tables, const int32_t* context_lens,
                            void* out, void* workspace, size_t workspace_bytes,
                            int32_t batch, int32_t num_heads, int32_t num_kv_heads,
                            int32_t head_dim, int32_t block_size, int32_t max_blocks,
                            int32_t num_blocks, float scale, int32_t chunk, int32_t dtype);

/*
 * The same call with its launches selectable.  NVJ_PHASE_SPLITK: the attention
 * kernel (all there is for chunk == 0 and NVJ_CHUNK_WHOLE_SEQUENCE; for chunk
 * > 0 the partials stay in `workspace`).  NVJ_PHASE_COMBINE: the second pass of
 * the fixed split (reads the partials an earlier split-K launch with the same
 * arguments left in `workspace`; nothing for the other modes).
 * NVJ_PHASE_CLEAR_COUNTERS: chunk == 0 only, set the counter region at the head
 * of `workspace` to zero first.  The balanced kernel needs the counters zero
 * when it starts and leaves them zero when it ends, so a caller that keeps one
 * workspace per stream clears it once (this bit alone, or with the first call)
 * and then passes NVJ_PHASE_SPLITK only: one launch per call.  Calls of
 * different shapes must not share such a workspace (the counter region of one
 * shape overlaps the partials of another; nvj_paged_decode_launch_counters keeps
 * the two apart).  A counter that was not zero is noticed by the wave that finds
 * more arrivals than the row has pieces: it sets word 0 of the counter region
 * (the stale flag; sticky until the region is cleared) to 1, puts the counter
 * back to zero and leaves that row of `out` unwritten.  Every kernel still ends
 * normally (never a fault, never a wait); a caller that cannot rule the
 * condition out reads the flag back after the call.  All three bits =
 * nvj_paged_decode_launch.  Same reference counterpart as
 * nvj_paged_decode_launch.
 *
 * NVJ_PHASE_SHARED_ROWS, or-ed in, keeps the balanced split from dealing whole
 * rows (see chunk == 0 above): the equal cut with shared rows is taken whatever
 * the lengths.  Same results to the same tolerance; a measurement and test aid.
 *
 * NVJ_PHASE_VALU_PRODUCTS, or-ed in, runs a measurement variant of the split-K
 * kernel that computes Q.K and P.V with vector-ALU dot products instead of the
 * matrix cores, so that the choice between the two can be timed on any
 * workload.  Same results to the same tolerance; never selected by default.
 * Exists for head_dim 128, bf16, exactly 4 or 8 query heads per KV head, a
 * multiple of 8 KV heads and chunk 0 or NVJ_CHUNK_WHOLE_SEQUENCE; anything else
 * returns NVJ_ERR_UNSUPPORTED.
 *
 * NVJ_PHASE_LOADS_ONLY, or-ed in, runs a second measurement variant: the same
 * page walk and K/V loads with no arithmetic behind them, so that the time of
 * the memory stream alone can be set against the real kernel's.  `out` receives
 * meaningless finite values.  head_dim 128, bf16, chunk 0 or
 * NVJ_CHUNK_WHOLE_SEQUENCE; anything else returns NVJ_ERR_UNSUPPORTED.
 */
#define NVJ_PHASE_SPLITK  1u
#define NVJ_PHASE_COMBINE 2u
#define NVJ_PHASE_VALU_PRODUCTS 4u
#define NVJ_PHASE_CLEAR_COUNTERS 8u
#define NVJ_PHASE_LOADS_ONLY 16u
#define NVJ_PHASE_SHARED_ROWS 32u
NVJ_API int nvj_paged_decode_launch_phases(void* stream,
                            const void* q, const void* k_cache, const void* v_cache,
                            const int32_t* block_tables, const int32_t* context_lens,
                            void* out, void* workspace, size_t workspace_bytes,
                            int32_t batch, int32_t num_heads, int32_t num_kv_heads,
                            int32_t head_dim, int32_t block_size, int32_t max_blocks,
                            int32_t num_blocks, float scale, int32_t chunk, int32_t dtype,
                            uint32_t phases);

/*
 * The balanced split (chunk == 0) as ONE launch with its counter region and its
 * partials in separate buffers, so that calls of any shapes can share both: a
 * counter region stays zero between calls whatever the shapes were.  Stands in
 * for the same reference call as nvj_paged_decode_launch
 * (layers/attention.py:389-397); it is the form an XLA custom call uses, with
 * `partials` an XLA-owned scratch result and counters == NULL.
 *
 *   partials  >= nvj_paged_decode_workspace_bytes(.., chunk 0)
 *                - nvj_paged_decode_counter_bytes(..) bytes, 16-byte aligned,
 *                contents need not be initialised
 *   counters  >= nvj_paged_decode_counter_bytes(..) bytes of int32, ZERO before
 *                the first call (nvj_paged_decode_counters_reset) and left zero
 *                by every call; or NULL: the library's own region is used, one
 *                per GPU, 64 KiB (batch * num_kv_heads < 16384, else
 *                NVJ_ERR_SCRATCH_LIMIT), zero when the library is loaded
 *
 *   phases    NVJ_PHASE_SPLITK for the call as described; NVJ_PHASE_CLEAR_COUNTERS
 *                or-ed in clears the counter region first (a second launch);
 *                the measurement bits of nvj_paged_decode_launch_phases apply
 *
 * Calls that may overlap in time on one GPU must not share a counter region
 * (with NULL: all such calls, and nvj_paged_decode_static_launch, share the
 * library's): an overlap loses rows of both calls, and is reported through the
 * stale flag (word 0 of the region) on a best-effort basis.
 *
 * nvj_paged_decode_counters_reset: enqueue a kernel (recordable into a graph)
 * that sets `counter_bytes` bytes at `counters` to zero, stale flag included;
 * counters == NULL: the library's own region of the current device.
 *
 * nvj_paged_decode_library_counters: device address and size of the library's
 * own region on the current device, for a caller that wants to read the stale
 * flag (its first int32) back.  No launch.
 */
NVJ_API int nvj_paged_decode_launch_counters(void* stream,
                            const void* q, const void* k_cache, const void* v_cache,
                            const int32_t* block_tables, const int32_t* context_lens,
                            void* out, void* partials, size_t partial_bytes,
                            void* counters, size_t counter_bytes,
                            int32_t batch, int32_t num_heads, int32_t num_kv_heads,
                            int32_t head_dim, int32_t block_size, int32_t max_blocks,
                            int32_t num_blocks, float scale, int32_t dtype, uint32_t phases);
NVJ_API int nvj_paged_decode_counters_reset(void* stream, void* counters, size_t counter_bytes);
NVJ_API int nvj_paged_decode_library_counters(void** counters, size_t* bytes);

/*
 * nvj_paged_decode_launch with chunk == 0 (balanced split) for callers that
 * cannot allocate device memory: code running under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the
 * reference (whose arrays are all allocated by XLA); results are those of
 * nvj_paged_decode_launch(chunk = 0) bit for bit.
 *
 * The split-K partials and counters live in a device array of
 * NVJ_STATIC_SCRATCH_BYTES that is part of the library image: every GPU the
 * library runs on holds its own copy from the first call on that GPU until the
 * process ends.  Its first 64 KiB are the library's own counter region (see
 * nvj_paged_decode_launch_counters): zero when the library is loaded and left
 * zero by every launch, so the call is a single kernel launch.  The call itself
 * allocates and frees nothing (no hipMalloc / hipFree, no allocating library
 * routine); the first call on a device looks the array's address up once.  The
 * device that `stream` belongs to must be the current device.
 *
 * A problem whose partials (nvj_paged_decode_workspace_bytes(..., chunk 0) minus
 * nvj_paged_decode_counter_bytes) exceed NVJ_STATIC_SCRATCH_BYTES - 64 KiB, or
 * whose counter region exceeds 64 KiB (batch * num_kv_heads >= 16384), is rejected with
 * NVJ_ERR_SCRATCH_LIMIT; batch 256 with 32 query heads of 128 dims needs 8.5 MB.  All calls on one GPU
 * share the one array: calls that may overlap in time on the same GPU (two
 * streams, two threads) race on it and must be serialised by the caller; calls
 * on one stream are ordered and safe.  Such a race, or context_lens rewritten
 * while the kernel runs, can also leave counters of the region non-zero, which
 * spoils later calls too (rows lost, stale flag set) until
 * nvj_paged_decode_counters_reset(stream, NULL, 0) has run.  Apart from the
 * counters being zero, nothing in the array has to survive from one call to
 * the next.
 */
#define NVJ_STATIC_SCRATCH_BYTES (16u << 20)
NVJ_API int nvj_paged_decode_static_launch(void* stream,
                            const void* q, const void* k_cache, const void* v_cache,
                            const int32_t* block_tables, const int32_t* context_lens,
                            void* out, int32_t batch, int32_t num_heads, int32_t num_kv_heads,
                            int32_t head_dim, int32_t block_size, int32_t max_blocks,
                            int32_t num_blocks, float scale, int32_t dtype);

/*
 * Fused per-head QK-RMSNorm + rotary embedding + KV-cache store: everything the
 * reference runs between the QKV projection and the attention call, in one
 * launch.  Replaces q_norm / k_norm (models/qwen3.py:157-160,
 * layers/layernorm.py:31-48), rotary_emb (models/qwen3.py:163,
 * layers/rotary_embedding.py:13-37, 96-106), the cast of q to the cache dtype
 * (layers/attention.py:386-387) and store_kv_to_cache (layers/attention.py:42-77).
 *
 *   qkv            [num_tokens, qkv_row_stride] bf16: per token the
 *                  num_heads q heads, then num_kv_heads k heads, then
 *                  num_kv_heads v heads, head_dim each (the fused projection
 *                  output, models/qwen3.py:147-155); qkv_row_stride in elements
 *   positions      [num_tokens] int32, clamped into [0, max_position)
 *   cos_sin_cache  [max_position, head_dim] f32: cos of the head_dim/2
 *                  frequencies, then sin (layers/rotary_embedding.py:60-76)
 *   q_norm_weight, k_norm_weight  [head_dim] f32, or both NULL for no QK norm
 *                  (the reference norms only when there is no QKV bias,
 *                  models/qwen3.py:125-131)
 *   slot_mapping   [num_tokens] int32; < 0 skips the token's K/V, >= num_slots
 *                  drops it (q_out is written for every token)
 *   k_cache, v_cache [num_slots, num_kv_heads, head_dim] bf16, updated in place
 *   q_out          [num_tokens, num_heads, head_dim] bf16
 *
 * Arithmetic: the fixed IEEE fp32 sequence documented at the top of
 * csrc/qk_norm_rope_store.hip (xor-butterfly sum of squares, exact 1/sqrt,
 * normalised value rounded to bf16 before the rotation, rotation in fp32,
 * result rounded to nearest-even bf16).  head_dim must be 128.
 */
NVJ_API int nvj_qk_norm_rope_store_launch(void* stream,
                            const void* qkv, int64_t qkv_row_stride,
                            const int32_t* positions, const float* cos_sin_cache,
                            int32_t max_position, const float* q_norm_weight,
                            const float* k_norm_weight, float eps,
                            const int32_t* slot_mapping, void* k_cache, void* v_cache,
                            void* q_out, int32_t num_tokens, int32_t num_heads,
                            int32_t num_kv_heads, int32_t head_dim, int64_t num_slots);

/*
 * Advance the device-resident metadata of a decode batch by one step, in
 * place.  Replaces the per-step host rebuild and upload of
 * ModelRunner._prepare_decode (engine/model_runner.py:334-376): once a step has
 * produced next_tokens[i] for every sequence, sequence i grows by that token and
 *
 *   input_ids[i]    = next_tokens[i]                         (seq.last_token)
 *   positions[i]    = len - 1
 *   context_lens[i] = len                                    (len = old length + 1)
 *   slot_mapping[i] = block_tables[i, (len-1) / block_size] * block_size
 *                     + (len-1) % block_size
 *                     (= block_table[-1] * block_size + last_block_num_tokens - 1)
 *
 * next_tokens is int32 (token_bytes 4) or int64 (token_bytes 8); all other
 * arrays are int32 [batch], block_tables int32 [batch, max_blocks].  The host
 * keeps block_tables current: when a sequence is about to enter a new page the
 * page number must be in its row before this call (the reference allocates it
 * in BlockManager.may_append, engine/block_manager.py:215-243).  A row with
 * context_lens <= 0 is inactive and stays so; a row whose next page is missing
 * (-1 padding or beyond max_blocks) is left unchanged; both get slot -1, i.e.
 * their K/V are not stored.
 */
NVJ_API int nvj_advance_decode_launch(void* stream, const void* next_tokens,
                            int32_t token_bytes, int32_t* input_ids, int32_t* positions,
                            int32_t* context_lens, int32_t* slot_mapping,
                            const int32_t* block_tables, int32_t batch, int32_t max_blocks,
                            int32_t block_size);

/*
 * Variable-length causal prefill attention over packed rows.  Replaces
 * variable_length_attention_prefill (layers/attention.py:135-279) as called
 * from Attention._prefill_attention (layers/attention.py:331-364).
 *
 *   q   [total_q_tokens, num_heads, head_dim]     `dtype`: NVJ_DTYPE_BF16 or NVJ_DTYPE_F16
 *   k,v [total_k_tokens, num_kv_heads, head_dim]  `dtype` (total_k_tokens =
 *       cu_seqlens_k[batch]); the new rows of the prompts, not the paged cache
 *   cu_seqlens_q, cu_seqlens_k [batch + 1] int32, device memory
 *   out [total_q_tokens, num_heads, head_dim]     `dtype`
 *
 * Sequence i owns q rows [cu_q[i], cu_q[i+1]) and k/v rows [cu_k[i], cu_k[i+1]).
 * Query position p (counted from the start of its sequence) attends key
 * positions <= p of the same sequence (the reference's q_pos >= k_pos mask,
 * :232-243, combined with the padding masks); query head h uses kv head
 * h / (num_heads / num_kv_heads); fp32 softmax and accumulation, probabilities
 * rounded to `dtype` for the PV product, result in `dtype`.  A query row with no visible
 * key (its sequence has no k rows) gives zeros.  The static max_seqlen_q /
 * max_seqlen_k of the reference are not needed: nothing is padded.
 * total_q_tokens bounds the launch and must be >= cu_seqlens_q[batch].
 * head_dim must be 128, scale >= 0.
 */
NVJ_API int nvj_prefill_attention_launch(void* stream, const void* q, const void* k,
                            const void* v, const int32_t* cu_seqlens_q,
                            const int32_t* cu_seqlens_k, void* out,
                            int32_t total_q_tokens, int32_t batch, int32_t num_heads,
                            int32_t num_kv_heads, int32_t head_dim, float scale, int32_t dtype);

/*
 * The same attention with keys and values read from the block-paged cache:
 * prompt rows behind a cached prefix (prefix caching, chunked prefill).  The
 * reference prepares exactly this call - cu_seqlens_k > cu_seqlens_q and
 * block_tables in the prefill context (engine/model_runner.py:286-312,
 * utils/context.py:129-166) - but its attention (layers/attention.py:331-364)
 * is handed only the new rows and never reads the cached part; this entry point
 * is what that context describes.  Run it after the store of the new rows.
 *
 *   q   [total_q_tokens, num_heads, head_dim]                     `dtype`
 *   k_cache, v_cache [num_blocks, block_size, num_kv_heads, head_dim]  `dtype`
 *   block_tables [batch, max_blocks] int32 (entries of live pages in [0, num_blocks))
 *   cu_seqlens_q, cu_seqlens_k [batch + 1] int32; len_k = cu_k[i+1] - cu_k[i] counts
 *       the keys of sequence i, cached and new together (clamped to
 *       max_blocks * block_size), as the reference's filler sets it (:288-291)
 *   out [total_q_tokens, num_heads, head_dim]                     `dtype`
 *
 * The len_q = cu_q[i+1] - cu_q[i] query rows of sequence i are its LAST len_q
 * positions: row j attends key positions <= len_k - len_q + j.  With
 * len_k == len_q this is nvj_prefill_attention_launch on the rows just
 * stored, bit for bit.  head_dim 128, block_size a multiple of 32, scale >= 0.
 */
NVJ_API int nvj_paged_prefill_attention_launch(void* stream, const void* q, const void* k_cache,
                            const void* v_cache, const int32_t* block_tables,
                            const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k, void* out,
                            int32_t total_q_tokens, int32_t batch, int32_t num_heads,
                            int32_t num_kv_heads, int32_t head_dim, int32_t block_size,
                            int32_t max_blocks, int32_t num_blocks, float scale, int32_t dtype);

/*
 * RMSNorm over the last dimension, optionally fused with the residual add.
 * Replaces RMSNorm._rms_forward (layers/layernorm.py:31-48) when `residual` is
 * NULL and RMSNorm._add_rms_forward (layers/layernorm.py:50-79) otherwise, as
 * called around every attention and MLP block (models/qwen3.py:305-313, 364).
 *
 *   x            [num_tokens, hidden] bf16
 *   residual     [num_tokens, hidden] bf16 or NULL
 *   weight       [hidden] float32
 *   y            [num_tokens, hidden] bf16: bf16((s * rsqrt(mean(s^2) + eps)) * weight)
 *   residual_out [num_tokens, hidden] bf16: bf16(s); NULL exactly when residual is
 *
 * with s = float(x) + float(residual) (or float(x)); the mean is taken over the
 * unrounded fp32 sums, as the reference does.  residual_out may be the same
 * buffer as residual; x and y must not overlap any other argument.  hidden must
 * be a multiple of 8 and at most 8192; all pointers 16-byte aligned.
 */
NVJ_API int nvj_add_rms_norm_launch(void* stream, const void* x, const void* residual,
                            const float* weight, float eps, void* y, void* residual_out,
                            int32_t num_tokens, int32_t hidden);

/*
 * SiLU(gate) * up for the fused gate/up projection of the MLP.  Replaces
 * SiluAndMul.__call__ (layers/activation.py:22-33; called at
 * models/qwen3.py:229).
 *
 *   x [num_tokens, x_row_stride] bf16: gate in columns [0, intermediate), up in
 *     [intermediate, 2 * intermediate) of every row (x_row_stride >= 2 *
 *     intermediate elements, a multiple of 8)
 *   y [num_tokens, intermediate] bf16
 *
 * Evaluated in fp32 from the bf16 inputs and rounded once to bf16 (the reference
 * leaves the rounding points of the bf16 expression to XLA).  intermediate must
 * be a multiple of 8; pointers 16-byte aligned.
 */
NVJ_API int nvj_silu_and_mul_launch(void* stream, const void* x, int64_t x_row_stride,
                            void* y, int32_t num_tokens, int32_t intermediate);

#ifdef __cplusplus
}  /* extern "C" */
#endif
#endif  /* NVJ_PAGED_ATTN_H_ */
