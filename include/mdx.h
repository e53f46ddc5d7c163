/*
 * mdx.h -- C ABI of libmdx.so: the block-diffusion attention hot path of the
 * nano_dvlm engine (opendatalab/MinerU-Diffusion) as hand-written gfx950 HIP
 * kernels for one MI355X.
 *
 * The reference has no FFI: its hot path is reached through Python call sites.
 * Each entry point below names the reference interface it stands in for.  All
 * pointers are BORROWED DEVICE pointers (the caller keeps the memory alive
 * until the stream has passed the call); outputs and workspaces are allocated
 * by the caller.  No entry point allocates, frees or synchronises; every
 * kernel is enqueued on `stream` (a hipStream_t, 0 = the null stream), so all
 * of them may be recorded into a HIP graph.
 *
 * Global state of the library, all of it: (1) a thread-local error string
 * (mdx_last_error); (2) per device, set once on the first call that needs it
 * and never changed afterwards: the raised dynamic-LDS limit of the staircase
 * pair kernel (a function attribute) and the number of compute units that the
 * paged attention sizes its splits by; (3) the file-scope __device__ array of
 * 40 MiB behind mdx_paged_block_attn_static, one copy per GPU, with the
 * per-device address of it cached after the first call on that device; calls
 * of that one entry point that overlap on one GPU race on the array.  No other
 * entry point shares memory between calls: they are re-entrant.
 *
 * Return value: 0 on success, a negative MDX_E* code otherwise (nothing has
 * been enqueued then); mdx_last_error() gives the reason as text.
 */
#ifndef MDX_H
#define MDX_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MDX_VERSION 100            /* major*10000 + minor*100 + patch */

#define MDX_OK            0
#define MDX_EINVAL       -1        /* bad argument: null pointer, negative size */
#define MDX_EUNSUPPORTED -2        /* shape / dtype / stride outside what the kernels cover */
#define MDX_EWORKSPACE   -3        /* workspace missing or too small */
#define MDX_ELAUNCH      -4        /* the HIP runtime refused the launch */

#define MDX_BF16 0                 /* q/k/v/o, the caches, the layer ops, the logits */
#define MDX_F16  1                 /* q/k/v/o and the caches of the two attention calls, the logits */
#define MDX_F32  2                 /* the logits; q/k/v/o and the caches of the two attention calls (fp32 arithmetic) */

typedef void* mdx_stream_t;        /* hipStream_t */

int         mdx_version(void);
const char* mdx_last_error(void);  /* thread-local; valid until the next failing call on this thread */

/*
 * store_kvcache -- replaces store_kvcache / store_kvcache_kernel
 * (engines/nano_dvlm/nanovllm/layers/attention.py:10-40; 4-D form
 * layers/sdar_attention.py:11-16 is the same call on flattened views).
 *
 * For token i in [0, n_tokens): slot = slot_mapping[i]; if slot == -1 skip,
 * else copy row_elems elements key + i*k_row_stride -> k_cache + slot*row_elems
 * and value + i*v_row_stride -> v_cache + slot*row_elems.  Strides are in
 * elements; rows themselves are dense (attention.py:36-38).  elem_size is in
 * bytes (2 for bf16/f16).  Slots outside [0, num_slots) are skipped instead
 * of written (the reference leaves them undefined); num_slots = pages*page.
 * If two tokens name the same slot the result holds one of the two rows.
 */
int mdx_store_kvcache(const void* key, const void* value,
                      int64_t k_row_stride, int64_t v_row_stride,
                      void* k_cache, void* v_cache,
                      const int32_t* slot_mapping,
                      int64_t n_tokens, int64_t row_elems, int32_t elem_size,
                      int64_t num_slots, mdx_stream_t stream);

/*
 * Staircase block-prefill attention over packed variable-length sequences --
 * replaces sparse_attn_varlen / sparse_attn_varlen_v2
 * (engines/nano_dvlm/nanovllm/kernels/triton/attention/block_prefill_attention_v2.py:16-202).
 *
 * q,o [total_tokens, Hq, d]; k,v [total_tokens, Hkv, d]; the innermost stride
 * is 1, token and head strides are given in elements (so the strided views of
 * a fused QKV projection are read in place; the reference copies them,
 * :182).  q, k, v, o 16-byte aligned; strides of q, k, v multiples of 8
 * elements, those of o multiples of 4 (multiples of 8 let the kernels write
 * whole 256-byte rows of o, the faster form).  cu_seqlens_q / cu_seqlens_k [batch+1] int32 device arrays; the
 * kernel is a self-attention and reads the sequence bounds from cu_seqlens_k,
 * like the reference (:48-50); both must describe the same sequences.
 * Blocks of staircase_size tokens (1,2,..,128) are right-aligned in every
 * sequence (:52-53, :98-102): query i sees key j iff
 * j <= ((i+pad)/S+1)*S-1-pad, pad = ceil(L/S)*S-L.  Hq % Hkv == 0 and
 * kv head = q head / (Hq/Hkv) (:34).  softmax(q k^T * scale) v with fp32
 * accumulation.  max_seqlen MUST be >= the longest sequence in cu_seqlens: it
 * sizes the grid, and rows of a longer sequence beyond it are never computed
 * (their o rows keep what they held; the lengths are on the device, so the
 * call cannot check this).  total_tokens is always a valid bound; the
 * reference interface has no such argument.  Supported: the reference kernel
 * takes q's dtype (:179-197) and BLOCK_DMODEL = head_dim (:183).  MDX_BF16 and
 * MDX_F16 with d a multiple of 16 up to 128 run on the 16-bit matrix
 * instructions (both the same kernels, fp16 within a few percent of bf16;
 * widths below 128 run as 128 with zero padding, in the one-head-per-wavefront
 * kernel, and only d columns of o are written; tensors 16-byte aligned with
 * strides that are multiples of 8 elements, o's of 4).  MDX_F32, and 16-bit
 * tensors whose d is another multiple of 4 up to 256, run in fp32 arithmetic
 * on the fp32 matrix instruction (probabilities never rounded, 16-bit inputs
 * widened; exact rather than fast: about a tenth of the 16-bit kernels' rate;
 * tensors aligned to four elements with strides that are multiples of 4).
 */
int mdx_staircase_attn_varlen(const void* q, const void* k, const void* v, void* o,
                              int64_t q_stride_t, int64_t q_stride_h,
                              int64_t k_stride_t, int64_t k_stride_h,
                              int64_t v_stride_t, int64_t v_stride_h,
                              int64_t o_stride_t, int64_t o_stride_h,
                              const int32_t* cu_seqlens_q, const int32_t* cu_seqlens_k,
                              int32_t batch, int32_t max_seqlen, int64_t total_tokens,
                              int32_t num_q_heads, int32_t num_kv_heads, int32_t head_dim,
                              int32_t staircase_size, float scale, int32_t dtype,
                              mdx_stream_t stream);

/*
 * Paged single-block ("decode") attention -- replaces the call
 * flash_attn_with_kvcache(q, k_cache, v_cache, cache_seqlens=, block_table=,
 * softmax_scale=, causal=False) of
 * engines/nano_dvlm/nanovllm/layers/sdar_attention.py:48-56 (flash-attn 2.8.3,
 * third party; inputs built by engine/model_runner.py:121-125,169-185).
 *
 * q,o [bs, Sq, Hq, d] with strides (q_stride_b, q_stride_s, q_stride_h, 1);
 * caches [num_pages, page_size, Hkv, d] with strides (cache_stride_page,
 * cache_stride_tok, cache_stride_head, 1); block_table [bs, max_pages] int32,
 * row stride bt_stride, entries past ceil(ctx/page_size) are not read (-1
 * padding, model_runner.py:123); context_lens [bs] int32.  Every query of
 * sequence b sees keys 0..context_lens[b]-1 (non-causal).  Rows with
 * context_lens[b] == 0 (graph padding, model_runner.py:205-208) produce
 * zeros.  Page ids outside [0, num_pages) are treated as holding no keys; a
 * sequence whose pages are all invalid therefore also produces zeros.
 * The workspace holds the split-KV partial results (and the split size when the
 * kernel picks it from the lengths); its size comes from
 * mdx_paged_block_attn_workspace_bytes with the same shape arguments, and its
 * contents need no initialisation.
 * Supported: Sq <= 128 (blocks longer than 32 positions run as tiles of 32 queries that stream the same keys), any Hq
 * that is a multiple of Hkv, page_size % 32 == 0.  MDX_BF16 and MDX_F16 with d a multiple of 16 up to 128 run on the
 * 16-bit matrix instructions (narrower heads are padded with zeros on the way into LDS; the partials keep their
 * 128-wide layout).  MDX_F32, and 16-bit tensors whose d is another multiple of 4 up to 256 (flash-attn takes heads
 * of up to 256 columns), run in fp32 arithmetic on the fp32 matrix instruction: one workgroup per (sequence, query head,
 * query tile) walks the whole context, no split over workgroups and no workspace (the workspace query returns 0 for those widths; a
 * workspace that is passed anyway is ignored); exact rather than fast.
 */
int64_t mdx_paged_block_attn_workspace_bytes(int32_t bs, int32_t sq, int32_t num_q_heads,
                                             int32_t num_kv_heads, int32_t head_dim,
                                             int32_t max_pages, int32_t page_size);
int mdx_paged_block_attn(const void* q, void* o, const void* k_cache, const void* v_cache,
                         int64_t q_stride_b, int64_t q_stride_s, int64_t q_stride_h,
                         int64_t o_stride_b, int64_t o_stride_s, int64_t o_stride_h,
                         int64_t cache_stride_page, int64_t cache_stride_tok, int64_t cache_stride_head,
                         const int32_t* block_table, int64_t bt_stride, const int32_t* context_lens,
                         int32_t bs, int32_t sq, int32_t num_q_heads, int32_t num_kv_heads,
                         int32_t head_dim, int32_t max_pages, int32_t page_size, int64_t num_pages,
                         float scale, int32_t dtype,
                         void* workspace, int64_t workspace_bytes, mdx_stream_t stream);

/*
 * The same in ONE launch where that pays: with about a (sequence, head group) pair per CU or
 * more, where only sequences far longer than the rest are split, the last split of a pair to
 * finish merges the pair's partials itself instead of a second (combine) launch; no workgroup
 * waits for another.  In a decode pass whose sequences stay whole (the usual case at batch 32)
 * this saves the launch of a kernel that finds nothing to do, 28 times per forward pass.  With
 * fewer pairs, where every sequence is split, the call makes the same two launches as
 * mdx_paged_block_attn (counting in costs each split workgroup a device-wide release).
 *
 * counters: mdx_paged_block_attn_counter_bytes(bs, Hq, Hkv) bytes of device memory (one fp32 per
 * sequence, head group and tile of 32 queries, sized for Sq = 128), 4-byte
 * aligned, that MUST BE ZERO before the first call and are left zero by every call that
 * completes; calls that may run at the same time (different streams) need counters of their
 * own.  workspace as above.  Same results bit for bit as mdx_paged_block_attn.
 */
int64_t mdx_paged_block_attn_counter_bytes(int32_t bs, int32_t num_q_heads, int32_t num_kv_heads);
int mdx_paged_block_attn_single_launch(const void* q, void* o, const void* k_cache, const void* v_cache,
                                       int64_t q_stride_b, int64_t q_stride_s, int64_t q_stride_h,
                                       int64_t o_stride_b, int64_t o_stride_s, int64_t o_stride_h,
                                       int64_t cache_stride_page, int64_t cache_stride_tok, int64_t cache_stride_head,
                                       const int32_t* block_table, int64_t bt_stride, const int32_t* context_lens,
                                       int32_t bs, int32_t sq, int32_t num_q_heads, int32_t num_kv_heads,
                                       int32_t head_dim, int32_t max_pages, int32_t page_size, int64_t num_pages,
                                       float scale, int32_t dtype,
                                       void* workspace, int64_t workspace_bytes,
                                       void* counters, int64_t counter_bytes, mdx_stream_t stream);

/*
 * mdx_paged_block_attn for callers that CANNOT ALLOCATE (code under HIP graph capture without an
 * allocator, tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in
 * the reference, whose call sites allocate freely.  Same arguments, kernels and results (bit for
 * bit) as mdx_paged_block_attn, without the workspace: the split-KV partials go into a 40 MiB
 * device array that is part of the library image (each GPU the library runs on holds it until
 * the process ends).  Shapes whose partials need more (the size mdx_paged_block_attn_workspace_bytes
 * reports; 32 sequences x 16 heads with page tables of 17 pages need 32.5 MiB, 64 such sequences
 * 65 MiB) are refused with MDX_EWORKSPACE.
 * The call itself allocates and frees nothing; the first call on each device looks the array's
 * address up (hipGetSymbolAddress), so make that call outside graph capture.  All calls on one
 * GPU share the array: calls that may overlap (different streams) race on it; calls on one
 * stream do not.
 */
int mdx_paged_block_attn_static(const void* q, void* o, const void* k_cache, const void* v_cache,
                                int64_t q_stride_b, int64_t q_stride_s, int64_t q_stride_h,
                                int64_t o_stride_b, int64_t o_stride_s, int64_t o_stride_h,
                                int64_t cache_stride_page, int64_t cache_stride_tok, int64_t cache_stride_head,
                                const int32_t* block_table, int64_t bt_stride, const int32_t* context_lens,
                                int32_t bs, int32_t sq, int32_t num_q_heads, int32_t num_kv_heads,
                                int32_t head_dim, int32_t max_pages, int32_t page_size, int64_t num_pages,
                                float scale, int32_t dtype, mdx_stream_t stream);

/*
 * Vocabulary projection fused with confidence + argmax -- replaces, for rows that are only wanted for
 * the unmask step, ParallelLMHead.forward's F.linear(x, weight)
 * (engines/nano_dvlm/nanovllm/layers/embed_head.py:61-67) followed by Sampler.prepare without noise
 * (layers/sampler.py:11-22); the [rows, vocab] logits are never written.
 *
 * x [rows, hidden] and w [vocab, hidden], MDX_BF16, row strides in elements (multiples of 8, 16-byte
 * aligned bases); hidden a multiple of 128.  The logits x . w^T are accumulated in fp32 and rounded to
 * bf16, as the projection's output is in the reference; then x0[r] = first index of the row's maximum,
 * x0_p[r] = softmax(logits / T)[x0[r]].  temperatures (NULL = 1.0): row r uses entry
 * (row_ids ? row_ids[r] : r) / rows_per_temp, so that rows compacted out of [bs, block] keep their
 * sequence's temperature; row_ids may be NULL.  The workspace (mdx_lm_head_confidence_workspace_bytes,
 * 16-byte aligned, contents need no initialisation) holds one 16-byte record per row and 128-entry slice
 * of the vocabulary.  Two launches: the projection tiles, then one wavefront per row folding its records.
 */
int64_t mdx_lm_head_confidence_workspace_bytes(int64_t rows, int64_t vocab);
int mdx_lm_head_confidence(const void* x, int64_t x_row_stride, const void* w, int64_t w_row_stride,
                           const float* temperatures, int32_t rows_per_temp, const int64_t* row_ids,
                           int64_t* x0, float* x0_p,
                           int64_t rows, int64_t vocab, int64_t hidden,
                           void* workspace, int64_t workspace_bytes, mdx_stream_t stream);

/*
 * Confidence + argmax over the vocabulary -- replaces Sampler.prepare
 * (engines/nano_dvlm/nanovllm/layers/sampler.py:11-22).
 *
 * logits [rows, vocab] (row stride in elements, dtype MDX_BF16/F16/F32);
 * temperatures: one float per group of rows_per_temp consecutive rows
 * ([bs] with rows_per_temp = block length; sampler.py:13), or NULL for 1.0;
 * noise: optional [rows, vocab] fp32 added to logits/T before the argmax
 * (the Gumbel term of sampler.py:15-18, made an explicit input so the kernel
 * holds no RNG), or NULL for the plain argmax.  Outputs: x0[r] = first index
 * of the maximum (int64), x0_p[r] = softmax(logits/T)[x0[r]] (fp32).  A row
 * without any finite logit (all -inf) has no softmax: x0 = 0, x0_p = 0, so
 * that no selection rule commits it.
 * Workspace from mdx_confidence_argmax_workspace_bytes (may be 0 bytes: then
 * workspace may be NULL).
 */
int64_t mdx_confidence_argmax_workspace_bytes(int64_t rows, int64_t vocab);
int mdx_confidence_argmax(const void* logits, int64_t row_stride, int32_t dtype,
                          const float* temperatures, int32_t rows_per_temp,
                          const float* noise, int64_t noise_row_stride,
                          int64_t* x0, float* x0_p,
                          int64_t rows, int64_t vocab,
                          void* workspace, int64_t workspace_bytes, mdx_stream_t stream);

/*
 * Selection of the positions to commit -- replaces the CPU loop of
 * Sampler.forward (layers/sampler.py:32-54) and _select_transfer_index
 * (mineru_diffusion/modeling_mineru_diffusion.py:518-532) on the device.
 *
 * Per sequence b (block length S <= 1024): masked = tokens[b,:] == mask_token_id;
 * conf = masked ? x0_p : -inf; hi = conf > threshold (strict).  If
 * count(hi) >= k commit all of hi, else commit the min(k, count(masked)) most
 * confident masked positions (ties: lower position first; a position whose
 * x0_p is -inf is never committed, which lets a caller mark rows it has no
 * fresh confidence for).  k = 1 gives the
 * engine's rule (sampler.py:41-50), k = block/steps the HF rule (k = 0, which
 * its schedule reaches when a block has fewer positions than steps, commits
 * the positions above the threshold and no others).  Writes
 * transfer[b,p] (uint8 0/1), tokens[b,p] = x0[b,p] where committed (in place),
 * and count[b] = number committed (int32).
 */
int mdx_select_transfer(const int64_t* x0, const float* x0_p, int64_t* tokens,
                        int64_t mask_token_id, float threshold, int32_t k,
                        uint8_t* transfer, int32_t* count,
                        int32_t bs, int32_t block_len, mdx_stream_t stream);

/*
 * The whole unmask step: mdx_confidence_argmax over [bs*block_len, vocab]
 * followed by mdx_select_transfer, on one stream (sampler.py:24-61 without
 * the host round trip).  temperatures [bs] or NULL.
 */
int mdx_unmask_step(const void* logits, int64_t row_stride, int32_t dtype,
                    const float* temperatures, const float* noise, int64_t noise_row_stride,
                    int64_t* tokens, int64_t mask_token_id, float threshold, int32_t k,
                    int64_t* x0, float* x0_p, uint8_t* transfer, int32_t* count,
                    int32_t bs, int32_t block_len, int64_t vocab,
                    void* workspace, int64_t workspace_bytes, mdx_stream_t stream);

/*
 * The same two calls with the Gumbel noise of Sampler.prepare (layers/sampler.py:15-16:
 * gumbel = -log(Exponential(1)), added to logits / T before the argmax) drawn inside the kernel
 * instead of read from a tensor.  The draw is a pure function of (seed, offset, row, column):
 * Philox-4x32-10 with key = seed (low word, high word) and counter = (column / 4, row, offset low
 * word, offset high word), whose four 32-bit outputs serve columns 4*(column/4) .. +3; an output r
 * becomes u = ((r >> 9) + 1/2) / 2^23 and the noise is -ln(-ln u).  A caller gives every step
 * another offset (as it would advance a generator); offset_dev, when not NULL, points to an int64
 * on the device whose value is added to offset when the kernel runs, so that a replayed HIP graph
 * can step it; row_ids, when not NULL, gives per logits row the row coordinate to use (int64
 * [rows], on the device; values below 2^32), so that a caller who compacted its rows keeps the noise of the
 * uncompacted layout.  x0_p is the softmax of logits / T at the drawn token (without noise), as in
 * sampler.py:20-21.  mdx_gumbel_noise writes the noise tensor that these calls stand for
 * ([rows <= 65535, vocab] fp32): mdx_confidence_argmax with that tensor gives the same bits.
 */
int mdx_confidence_argmax_gumbel(const void* logits, int64_t row_stride, int32_t dtype,
                                 const float* temperatures, int32_t rows_per_temp,
                                 uint64_t seed, uint64_t offset, const int64_t* offset_dev, const int64_t* row_ids,
                                 int64_t* x0, float* x0_p, int64_t rows, int64_t vocab,
                                 void* workspace, int64_t workspace_bytes, mdx_stream_t stream);
int mdx_unmask_step_gumbel(const void* logits, int64_t row_stride, int32_t dtype,
                           const float* temperatures,
                           uint64_t seed, uint64_t offset, const int64_t* offset_dev, const int64_t* row_ids,
                           int64_t* tokens, int64_t mask_token_id, float threshold, int32_t k,
                           int64_t* x0, float* x0_p, uint8_t* transfer, int32_t* count,
                           int32_t bs, int32_t block_len, int64_t vocab,
                           void* workspace, int64_t workspace_bytes, mdx_stream_t stream);
int mdx_gumbel_noise(float* noise, int64_t noise_row_stride, int64_t rows, int64_t vocab,
                     uint64_t seed, uint64_t offset, const int64_t* offset_dev, const int64_t* row_ids,
                     mdx_stream_t stream);

/*
 * Top-k / top-p filtering of logits before sampling -- replaces top_k_logits and top_p_logits of the
 * HF variant (mineru_diffusion/modeling_mineru_diffusion.py:585-600), applied in the order of
 * sample_with_temperature_topk_topp (:608-611): out = logits with every element below the row's
 * cut-off value set to -inf, to be passed on to mdx_confidence_argmax / mdx_unmask_step (whose noise
 * input then samples from the filtered distribution as torch.multinomial does at :613).
 *
 * logits, out: [rows, vocab <= 2^23], MDX_BF16 or MDX_F16 (the cut-off is found by counting over the 65 536
 * values a 16-bit element can take; MDX_F32 is refused), row strides in elements; out may be logits
 * itself.  top_k = 0 (or >= vocab) switches the top-k filter off, top_p >= 1 the top-p filter.
 * top-k keeps the elements >= the k-th largest value (equal values are all kept, as in the reference);
 * top-p keeps, of what top-k kept and with probabilities softmax(kept / T), the elements >= the value at
 * which the cumulative probability taken from the largest element down first exceeds top_p (the
 * reference keeps that element too; among EQUAL values at the cut-off its sort order decides, here all
 * of them are kept).  temperatures as for mdx_confidence_argmax.  No workspace.
 */
int mdx_filter_logits(const void* logits, int64_t row_stride, int32_t dtype,
                      const float* temperatures, int32_t rows_per_temp,
                      int32_t top_k, float top_p,
                      void* out, int64_t out_row_stride,
                      int64_t rows, int64_t vocab, mdx_stream_t stream);

/*
 * Fused producer of the attention inputs for one decoder layer: per-head RMSNorm of q and k,
 * rotary embedding, and the KV-cache store, in one pass over the fused QKV projection output --
 * replaces the chain q_norm / k_norm / rotary_emb / store_kvcache of
 * engines/nano_dvlm/nanovllm/models/sdar.py:79-83 (layers/layernorm.py:16-26,
 * layers/rotary_embedding.py:6-14,37-48, layers/sdar_attention.py:37-38).
 *
 * qkv [n_tokens, (Hq + 2 Hkv) * d] (row stride in elements; heads laid out q | k | v);
 * q_weight, k_weight [d]; cos_table, sin_table [max_positions, d/2] fp32; positions [n_tokens]
 * int64.  Writes q_out [n_tokens, Hq, d] and, if non-null, k_out [n_tokens, Hkv, d] (the
 * rotated k the prefill attention reads), and, if the caches are given, the rotated k row and
 * the raw v row of token i into slot slot_mapping[i] (-1 and out-of-range slots skipped) of
 * k_cache / v_cache [num_slots, Hkv, d].  v itself stays where it is (a view of qkv).
 * Rounding follows the reference: normalise in fp32, round to bf16, multiply by the weight
 * in bf16, rotate in fp32, round once.  Supported: d == 128, MDX_BF16.
 */
int mdx_qk_norm_rope_store(const void* qkv, int64_t qkv_row_stride,
                           const void* q_weight, const void* k_weight, float eps,
                           const float* cos_table, const float* sin_table, int64_t max_positions,
                           const int64_t* positions,
                           void* q_out, int64_t q_out_row_stride,
                           void* k_out, int64_t k_out_row_stride,
                           void* k_cache, void* v_cache, const int32_t* slot_mapping, int64_t num_slots,
                           int64_t n_tokens, int32_t num_q_heads, int32_t num_kv_heads, int32_t head_dim,
                           int32_t dtype, mdx_stream_t stream);

/*
 * Residual add + RMSNorm of one decoder-layer input, one pass over the rows -- replaces
 * RMSNorm.forward of engines/nano_dvlm/nanovllm/layers/layernorm.py:16-51 as called at
 * nanovllm/models/sdar.py:147-152,180.
 *
 * x, out [rows, hidden]; weight [hidden]; row strides in elements.  With residual_in:
 * s = float(x) + float(residual_in); residual_out = round(s); out = round(s * rsqrt(mean(s^2) +
 * eps)) * weight, the product rounded again (add_rms_forward, :28-41).  With residual_in and
 * residual_out both NULL: the same with s = float(x) (rms_forward, :16-26).  out may alias x and
 * residual_out may alias residual_in.  Supported: MDX_BF16, hidden a multiple of 8 up to 8192.
 */
int mdx_add_rms_norm(const void* x, int64_t x_row_stride,
                     const void* residual_in, int64_t residual_in_row_stride,
                     void* residual_out, int64_t residual_out_row_stride,
                     const void* weight, float eps,
                     void* out, int64_t out_row_stride,
                     int64_t rows, int32_t hidden, int32_t dtype, mdx_stream_t stream);

/*
 * SiluAndMul.forward of engines/nano_dvlm/nanovllm/layers/activation.py:7-16 (called at
 * nanovllm/models/sdar.py:110-111): x [rows, 2 * intermediate] -> out [rows, intermediate] =
 * round(silu(float(x[:, :I]))) * x[:, I:], the product rounded again.  Row strides in
 * elements.  Supported: MDX_BF16, intermediate a multiple of 8.
 */
int mdx_silu_and_mul(const void* x, int64_t x_row_stride, void* out, int64_t out_row_stride,
                     int64_t rows, int32_t intermediate, int32_t dtype, mdx_stream_t stream);

/*
 * Denoising-block state kept on the device between decode passes (one entry per sequence of the
 * batch, "lane"): tokens [bs, block_len] int64 (the current block, mask_token_id where still masked),
 * lens [bs] (committed tokens), phase [bs] (MDX_PHASE_*), step [bs], step_map [bs, block_len].
 * With these three calls a decode pass is a fixed list of launches: no upload of pass inputs, no
 * blocking download of results; the host reads the 16-byte status of a lane when it wants to.
 */
#define MDX_PHASE_IDLE      0      /* padding lane or finished sequence: stores nothing, attends to nothing */
#define MDX_PHASE_DENOISING 1      /* block holds masked positions (SequenceStatus.RUNNING) */
#define MDX_PHASE_CACHING   2      /* block complete; the next pass stores its K/V (SequenceStatus.CACHING) */

/*
 * The pass inputs of ModelRunner.prepare_decode (engines/nano_dvlm/nanovllm/engine/model_runner.py:
 * 169-185) computed on the device: positions[b, p] = lens[b] + p, slot_mapping[b, p] =
 * block_table[b, t / page_size] * page_size + t % page_size with t = lens[b] + p (Sequence.get_slots,
 * engine/sequence.py:117-141; -1 where the page table has no page), context_lens[b] = lens[b] +
 * block_len.  Idle lanes get positions 0, slots -1, context 0 (the graph padding of
 * model_runner.py:203-208).
 */
int mdx_block_prepare(const int32_t* lens, const int32_t* phase,
                      const int32_t* block_table, int64_t bt_stride, int32_t max_pages,
                      int32_t page_size, int32_t block_len,
                      int64_t* positions, int32_t* slot_mapping, int32_t* context_lens,
                      int32_t bs, mdx_stream_t stream);

/*
 * rows_out[i] = flat index b * block_len + p of the i-th still-masked position of the denoising lanes,
 * in order; entries from the count up to rows_cap repeat entry 0 (0 when nothing is masked), so that
 * a consumer of fixed size rows_cap may process them all; *n_rows_out = the count (entries beyond
 * rows_cap are dropped: the caller sizes rows_cap from a bound it knows).  The sampler looks at the
 * logits of masked positions only (layers/sampler.py:39,54).
 */
int mdx_masked_rows(const int64_t* tokens, const int32_t* phase, int64_t mask_token_id,
                    int32_t bs, int32_t block_len,
                    int64_t* rows_out, int32_t rows_cap, int32_t* n_rows_out, mdx_stream_t stream);

/*
 * After mdx_select_transfer: the rest of Sampler.forward (layers/sampler.py:56-59: step_map[transfer] =
 * step, step += 1) and Scheduler.postprocess (engine/scheduler.py:65-82) per lane.  A denoising lane
 * whose block has no masked position left becomes caching; a caching lane (this pass has stored its
 * block's K/V) appends the block to out_tokens / out_steps [bs, out_stride] at offset lens - first_len
 * (Sequence.append_block, engine/sequence.py:97-101; positions at or beyond out_stride are dropped), adds block_len to lens, refills the block with
 * mask_token_id and becomes idle if the block held one of its n_stop stop_ids [bs, n_stop] (-1 = unused
 * entry) or lens - first_len >= max_new, else denoising again.  status [bs, 4] int32 = (phase, lens,
 * masked positions left, positions committed by this pass).
 */
int mdx_block_advance(int64_t* tokens, const uint8_t* transfer,
                      int32_t* step_map, int32_t* step, int32_t* phase, int32_t* lens,
                      const int32_t* first_len, const int32_t* max_new,
                      const int64_t* stop_ids, int32_t n_stop,
                      int64_t* out_tokens, int32_t* out_steps, int64_t out_stride,
                      int32_t* status, int64_t mask_token_id,
                      int32_t bs, int32_t block_len, mdx_stream_t stream);

/*
 * Calibration helper of bench.py -- no counterpart in the reference.  A register-only loop of back-to-back bf16
 * MFMAs (shape 32 = v_mfma_f32_32x32x16_bf16, 16 = v_mfma_f32_16x16x32_bf16) in `blocks` workgroups of four
 * wavefronts, `iters` (rounded up to a multiple of 8) x 8 (x 16) instructions per wavefront, on operands read once:
 * 64 uint32 per thread (blocks x 256 threads) holding bf16 pairs.  out: one float per thread.  What the matrix pipe
 * sustains on that data under the board's power limit; mdx_calib_mfma_loop_flops gives the flops of a launch.
 */
int64_t mdx_calib_mfma_loop_flops(int32_t shape, int32_t blocks, int32_t iters);
int mdx_calib_mfma_loop(int32_t shape, const void* operands, float* out, int32_t blocks, int32_t iters, mdx_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* MDX_H */
