/*
 * libcpmcu_amd -- C-ABI of the MI355X (gfx950) speculative-decoding verify/draft path.
 *
 * Two groups of entry points:
 *
 *  1. the model-level mirror of the reference's pybind module `cpmcu.C`
 *     (src/entry.cu:98-534): same names with a `cpmcu_` prefix, same parameter
 *     lists, `const char*` for the name and `uint64_t` for raw pointers.  State
 *     is one process-global model, as in the reference (src/entry.cu:98).
 *
 *  2. operator-level entry points for the four subsystems of the path, with
 *     explicit shapes, device pointers and a stream handle.  They have no
 *     counterpart at the reference's boundary; each cites the reference
 *     function whose work it does.
 *
 * Conventions
 *   - every function returns a status (CPMCU_OK = 0); on failure the message is
 *     available from cpmcu_last_error() (thread-local).  The Python shim maps
 *     CPMCU_ERR_INVALID_ARGUMENT to ValueError and everything else to
 *     RuntimeError, matching how std::invalid_argument / std::runtime_error
 *     cross pybind in the reference.
 *   - "device pointer" = HIP device memory owned by the caller for the duration
 *     of the call; "fp16" tensors are 16-bit floating point in the element type in
 *     force -- IEEE binary16 by default, bfloat16 under torch_dtype = 1 / the "dtype"
 *     option below -- row-major unless stated.
 *   - `stream` is a hipStream_t passed as void*; NULL selects the library's own
 *     blocking stream (the counterpart of calc_stream, src/utils.cu:6,19).
 *   - operator-level calls only enqueue work; they never synchronise.
 *
 * Paged KV cache layout (this library's own; the reference keeps flat
 * [budget, kv_heads*head_dim] buffers, src/model/kvcache.cuh:18-25, and its
 * layout never crosses the boundary):
 *   page size 256 tokens, head_dim 128.
 *   K pool  [num_pages][Hkv][256][128] fp16 -- one token's head row is 256 B.
 *   V pool  [num_pages][Hkv][128][256] fp16 -- transposed (dim-major) so that
 *           the P.V matrix product reads 8 consecutive tokens per lane; inside
 *           every aligned group of 16 tokens the slot of token t is
 *           (t & 3) | ((t & 4) << 1) | ((t & 8) >> 1)   (bits 2 and 3 swapped),
 *           which is the order in which the MFMA accumulator of Q.K^T hands
 *           the probabilities to the next MFMA.
 *   block_table[i] = physical page of logical page i (tokens 256i..256i+255);
 *   one table serves every layer, each layer has its own K and V pool.
 */
#ifndef CPMCU_AMD_H
#define CPMCU_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define CPMCU_OK 0
#define CPMCU_ERR_INVALID_ARGUMENT 1 /* -> ValueError  (std::invalid_argument in the reference) */
#define CPMCU_ERR_RUNTIME 2          /* -> RuntimeError (std::runtime_error) */
#define CPMCU_ERR_UNSUPPORTED 3      /* -> RuntimeError: entry point outside the verify/draft path */
#define CPMCU_ERR_HIP 4              /* -> RuntimeError: a HIP call failed */

/* flags of cpmcu_accept_commit, cpmcu_verify_tail_inplace and cpmcu_verify_step */
#define CPMCU_COMMIT_ADVANCE_LENGTH 1
#define CPMCU_COMMIT_NEXT_ROOT 2

#define CPMCU_PAGE_SIZE 256
#define CPMCU_HEAD_DIM 128
#define CPMCU_MAX_TREE 128

const char* cpmcu_last_error(void);
/* Library version string and the GPU architecture the kernels were built for. */
const char* cpmcu_version(void);

/* No reference counterpart: kernel-shape switches for tests and tuning (process-wide, not thread-safe
 * against concurrent calls).  Initial values come from the environment, read once when the library is
 * first used.
 *   "dtype"                 element type of every 16-bit floating-point tensor handed to the entry points from now on:
 *                           0 = IEEE half (default), 1 = bfloat16 -- the two types the reference builds its
 *                           templates for (src/entry.cu:26-59, torch_dtype).  Process-wide, like the reference's
 *                           model: cpmcu_init_base_model sets it from its torch_dtype, cpmcu_shutdown puts it
 *                           back to 0; the operator-level entry points follow whatever is in force.  Kernels
 *                           that only move values (append, compaction, gathers, weight tiling) do not care;
 *   "attn_kv_groups"        0 = chosen per call (default), 1 / 2 = force the 256-row / the two-KV-group
 *                           shape of the tree-attention kernel (CPMCU_ATTN_KV_GROUPS=1|2);
 *   "head_share_last_pass"  1 = the waves of a workgroup share the row blocks of a partly filled last pass
 *                           of the head GEMM (default), 0 = plain mapping (CPMCU_HEAD_NO_SHARE set);
 *   "head_stream_kernel"    1 = tiled head weights whose row blocks make at least one full pass over the GPU's
 *                           wave slots run the streaming GEMM kernel, on a multiple of the CU count in workgroups
 *                           (up to 1024) beyond four passes (two for 65 to 128 hidden rows) (default), 0 = always
 *                           the K-chunked kernel (CPMCU_HEAD_NO_STREAM set);
 *   "attn_merge_in_launch"  1 = the workgroups of a split tree-attention launch merge their own partials when the
 *                           launch fits the GPU's CUs and has at most 32 splits (default), 0 = always the separate
 *                           merge launch (CPMCU_ATTN_SEPARATE_MERGE set);
 *   "attn_merge_wait_us"    longest time a workgroup of such a launch waits for the others of its merge before it
 *                           leaves its share to the last one to arrive (default 2000; 0 = never wait);
 *   "topk_row_kernel"       1 = top-k by the one-launch row kernel (rows of more than 32768 elements in slices and a
 *                           merge of the slices' k best) (default), 0 = k rounds of a maximum search per chunk of 2048
 *                           elements and a merge launch, for chunks x k up to 2048: the same results, bit for bit,
 *                           from independent code. */
int cpmcu_set_option(const char* name, int value);

/* ------------------------------------------------------------------------- */
/* 1. Model-level mirror of src/entry.cu                                      */
/* ------------------------------------------------------------------------- */

/* src/entry.cu:100-136 init_base_model.  Records the target-model geometry.
 * torch_dtype: 0 = fp16, 1 = bf16 (src/entry.cu:26-59; anything else: "dtype not compiled", :43,52).  It becomes the
 * element type of every call that follows, model-level and operator-level, until cpmcu_shutdown. */
int cpmcu_init_base_model(float memory_limit, int vocab_size, int num_hidden_layers, int hidden_size,
                          int intermediate_size, int num_attention_heads, int num_key_value_heads,
                          int head_dim, float rms_norm_eps, int torch_dtype, int chunk_length,
                          float scale_embed, float scale_lmhead, float scale_residual);

/* src/entry.cu:278-301 init_eagle_model. */
int cpmcu_init_eagle_model(int num_layers, int num_iter, int topk_per_iter, int tree_size, int torch_dtype);

/* src/entry.cu:303-341 init_minicpm4_eagle_model (FR-Spec drafter over the base model). */
int cpmcu_init_minicpm4_eagle_model(int num_layers, int num_iter, int topk_per_iter, int tree_size,
                                    int torch_dtype, int apply_eagle_quant, int group_size,
                                    int eagle_window_size, int frspec_vocab_size, float residual_scale,
                                    int use_input_norm, int use_attn_norm);

/* src/entry.cu:462-464 init_storage: allocates lm_head, the FR-Spec sub-matrix,
 * the paged KV pools of every layer, the page table and scratch; writes the
 * maximum supported context (tokens) to *max_context. */
int cpmcu_init_storage(int* max_context);

/* src/entry.cu:466-468 load_model: blocking H2D copy of one named tensor from a
 * HOST pointer.  Names on this path: "lm_head.weight" ([vocab, hidden] fp16),
 * "eagle.token_id_remap" ([frspec_vocab] int32; must be loaded before
 * lm_head.weight, src/model/minicpm4/minicpm4_eagle.cuh:193-194,215-219).
 * Any other name -> CPMCU_ERR_INVALID_ARGUMENT (src/model/model.cuh:131-135). */
int cpmcu_load_model(const char* name, uint64_t host_ptr);

/* src/entry.cu:470-472 / :474-496 / :498-500.  prefill and decode need the dense
 * transformer layers and draft needs the EAGLE layer, none of which is part of
 * this path: they return CPMCU_ERR_UNSUPPORTED.  The parts of decode that are on
 * the path are cpmcu_decode_attention and cpmcu_decode_lm_head below. */
int cpmcu_prefill(int input_length, int history_length, uint64_t input, uint64_t position_ids, uint64_t output);
int cpmcu_decode(int input_length, int padded_length, uint64_t input, uint64_t position_ids,
                 uint64_t cache_length, uint64_t mask_2d, uint64_t output, int cuda_graph);
int cpmcu_draft(uint64_t tree_draft_ids, uint64_t tree_position_ids, uint64_t cache_length,
                uint64_t attn_mask, uint64_t tree_parent);

/* src/entry.cu:502-504 verify_and_fix -> MiniCPM4EagleImpl::verify
 * (src/model/minicpm4/minicpm4_eagle.cuh:398-418): greedy tree acceptance,
 * one stream synchronisation, compaction of the accepted rows in the K and V
 * pools of every layer, pred[0..a) <- accepted token ids.  All pointers are
 * device pointers; attn_mask has one uint64 per row (num_tokens <= 64, as at the
 * reference's boundary).  *accept_length receives a. */
int cpmcu_verify_and_fix(int num_tokens, uint64_t pred, uint64_t gt, uint64_t position_ids,
                         uint64_t cache_length, uint64_t attn_mask, uint64_t tree_parent,
                         int* accept_length);

/* One whole verify step on the model's storage, with the library's own HIP graph -- the part of
 * decode(..., cuda_graph = true) + verify_and_fix (src/entry.cu:474-496,502-504) that lies on the path: for
 * every layer the KV append of the num_tokens tree rows and the tree attention on the paged cache
 * (cpmcu_decode_attention), the target head with its arg-max (cpmcu_decode_lm_head without the logits), greedy
 * acceptance, compaction of every cache and the accepted ids (cpmcu_verify_and_fix) -- 34 launches for 32
 * layers.  The dense layers that produce q / k_new / v_new / hidden between those calls are outside the path,
 * so their outputs are inputs here.
 *   q, k_new, v_new, attn_out: HOST arrays [num_layers] (= num_hidden_layers) of device addresses: q[l] [T][Hq][128],
 *       k_new[l] / v_new[l] [T][Hkv*128], attn_out[l] like q[l];
 *   hidden [T][hidden_size]; draft_ids int32[T] (read only); position_ids int32[T]; cache_length int32[1] = P;
 *   kv_length int32[1] = P + T (the pre-incremented length of cpmcu/llm.py:272, kept as a scalar of its own so
 *       that neither is rewritten between the calls of a step); attn_mask uint64[T] for T <= 64 as in the reference,
 *       uint64[T][2] (word w of a row holds bits 64w..64w+63) for trees of 65 to CPMCU_MAX_TREE nodes, which the reference
 *       does not have; tree_parent int32[T];
 *   block_table: device int32[] logical -> physical pages to use for this step, or 0 = the model's table;
 *   outputs: gt_out int32[T] (0 = skip), accepted_ids int32[T] (first a entries), prev_hidden [T][hidden_size]
 *       (0 = skip: rows hidden[path[d]], src/model/eagle.cuh:108-115), next_position_ids int32[T] (0 = skip),
 *       result int32[1 + T] = (a, ids) in device or pinned host memory (0 = skip);
 *   flags: CPMCU_COMMIT_ADVANCE_LENGTH advances cache_length, kv_length and position_ids by a on the device
 *       (one more single-workgroup launch), so the next step of the same tree shape needs no host write.
 *   cuda_graph != 0: the step is captured once per (padded_length, num_tokens) -- the reference's key,
 *       src/entry.cu:476 -- and per set of addresses, and replayed afterwards (hipGraphLaunch); keep the buffers
 *       static, as cpmcu/llm.py does.  The call only enqueues on the library's stream: synchronise
 *       (cpmcu_synchronize) before reading results. */
int cpmcu_verify_step(int num_layers, int num_tokens, int padded_length, const uint64_t* q, const uint64_t* k_new, const uint64_t* v_new,
                      const uint64_t* attn_out, uint64_t hidden, uint64_t draft_ids, uint64_t position_ids,
                      uint64_t cache_length, uint64_t kv_length, uint64_t attn_mask, uint64_t tree_parent, uint64_t block_table,
                      uint64_t gt_out, uint64_t accepted_ids, uint64_t prev_hidden, uint64_t next_position_ids,
                      uint64_t result, int flags, int cuda_graph);

/* No reference counterpart (the reference captures decode only, src/entry.cu:475-492): the same graph mechanism
 * for any sequence of the model-level calls that only enqueue -- cpmcu_decode_attention, cpmcu_draft_attention,
 * cpmcu_decode_lm_head, cpmcu_draft_head, cpmcu_draft_round, cpmcu_draft_finish, cpmcu_verify_step with
 * cuda_graph = 0.  Calls made between capture_begin and capture_end are recorded on the library's stream instead
 * of run; capture_end hands back an id, cpmcu_graph_replay enqueues the recorded launches as one graph.  The
 * addresses passed during the capture are baked in; lengths are read from device memory at replay, as always. */
int cpmcu_capture_begin(void);
int cpmcu_capture_end(int* graph_id);
int cpmcu_graph_replay(int graph_id);
/* Frees a graph made by cpmcu_capture_end (its id may be handed out again); waits for the library's stream first. */
int cpmcu_graph_destroy(int graph_id);
/* No reference counterpart: how many captured verify steps (cpmcu_verify_step with cuda_graph = 1) the library holds.
 * It keeps at most 16 -- one per (padded_length, num_tokens), set of buffer addresses and option settings met -- and
 * drops the one unused the longest when another is needed (the reference keeps one, src/entry.cu:476-484). */
int cpmcu_step_graph_count(void);

/* src/entry.cu:506-508 print_perf_summary: prints the per-operator event timings
 * collected when CPMCU_PERF=1 is set in the environment. */
int cpmcu_print_perf_summary(void);

/* The slice of Attention::decode that is on the path (src/model/attn.cuh:199-229):
 * append the input_length new K/V rows of `layer` at cache rows
 * [cache_length - input_length, cache_length) and run tree attention over the
 * model's paged cache.  cache_length is the device scalar already incremented by
 * input_length, as cpmcu/llm.py:272 leaves it for the reference's flash call.
 *   q [input_length][Hq][D], k_new/v_new [input_length][Hkv*D], out like q.
 * mask_2d: uint64 per row, 0 = causal chain (no tree). */
int cpmcu_decode_attention(int layer, int input_length, int padded_length, uint64_t q, uint64_t k_new,
                           uint64_t v_new, uint64_t cache_length, uint64_t mask_2d, uint64_t out);

/* The same slice of Attention::decode for the drafter's own layer(s)
 * (src/model/minicpm4/minicpm4_eagle.cuh:247,359; src/model/eagle.cuh:188-233): they keep KV caches of
 * their own (minicpm4_eagle.cuh:76,183) and attend through the block sliding window
 * eagle_window_size given to init_minicpm4_eagle_model (Attention::window_size,
 * src/model/attn.cuh:228; see cpmcu_tree_attention_window).
 *   draft_layer: index into the drafter's num_layers layers.
 *   mask_2d / mask_k_range: Mask(eagle_mask_2d, k, k * d) of round d -- one uint64 per row whose bits
 *           refer to the last mask_k_range <= 64 keys; 0 / 0 = causal chain (the drafter's prefill of
 *           the accepted tokens, in chunks of <= 64 rows).
 * The accepted-path compaction of cpmcu_verify_and_fix does not touch these caches, as in the
 * reference (fix_kv_cache runs over the base model's caches only). */
int cpmcu_draft_attention(int draft_layer, int input_length, int padded_length, uint64_t q, uint64_t k_new,
                          uint64_t v_new, uint64_t cache_length, uint64_t mask_2d, int mask_k_range, uint64_t out);

/* LMHead::prefill on the loaded lm_head (src/model/linear.cuh:82-101,
 * src/model/model.cuh:164) plus the arg-max the reference leaves to PyTorch
 * (cpmcu/speculative/tree_drafter.py:153,233).  logits ([>=n][vocab] fp16) and
 * gt (int32[n]) may each be 0 to skip that output. */
int cpmcu_decode_lm_head(int input_length, uint64_t hidden, uint64_t logits, uint64_t gt);

/* FR-Spec draft head on the loaded sub-matrix: logits' = hidden . W'^T, log-softmax,
 * top-k, ids mapped back to the full vocabulary
 * (src/model/minicpm4/minicpm4_eagle.cuh:319-326,366-368).
 *   hidden [n][H]; out: topk_val [n][k] fp16 (log-probs), topk_pos [n][k] int32
 *   (FR-Spec indices), topk_ids [n][k] int32 (full-vocabulary ids). */
int cpmcu_draft_head(int n, uint64_t hidden, uint64_t topk_val, uint64_t topk_pos, uint64_t topk_ids);

/* draft() without the drafter's dense layers (src/model/minicpm4/minicpm4_eagle.cuh:304-396): what runs between
 * them, with the drafter's state (tried_history_*, eagle_mask_2d, running log-probs) kept by the library.
 *   cpmcu_draft_round(d, ...), d = 0 .. num_iter - 1 in order: FR-Spec head on hidden (1 row at d = 0: the last
 *       accepted row of the drafter's output, :320; topk_per_iter rows afterwards, :366), log-softmax, top-k, and the
 *       tree bookkeeping of the round (:321-332 / :367-382).  next_ids int32[topk_per_iter] out: the token ids to
 *       embed for the next round (full-vocabulary ids); parent_rows int32[topk_per_iter] out (d >= 1; may be 0): the
 *       row of the previous hidden states each pick continues (remap_hidden, :377); draft_mask uint64[topk_per_iter]
 *       out (may be 0): Mask(eagle_mask_2d, k, k * (d + 1)) for cpmcu_draft_attention of the next round.
 *   cpmcu_draft_finish (:385-393): tree_draft_ids[1 .. tree_size) (entry 0, the root, is the caller's),
 *       tree_position_ids / tree_attn_mask (one uint64 per row) / tree_parent [tree_size]; cache_length is the
 *       device scalar P (the reference copies it to the host first, :305; here it is read on the device).
 * Both only enqueue on the library's stream.  A round out of order or a finish before the last round is
 * CPMCU_ERR_INVALID_ARGUMENT. */
int cpmcu_draft_round(int d, uint64_t hidden, uint64_t next_ids, uint64_t parent_rows, uint64_t draft_mask);
int cpmcu_draft_finish(uint64_t tree_draft_ids, uint64_t tree_position_ids, uint64_t cache_length, uint64_t tree_attn_mask,
                       uint64_t tree_parent);

/* No reference counterpart: install a logical -> physical page permutation (host int32[n], distinct entries of
 * [0, num_pages)); the logical pages behind the n given ones take the remaining physical pages in ascending
 * order, so the table is always a permutation of all pages.  The default table is the identity. */
int cpmcu_set_block_table(const int32_t* host_table, int n);

/* No reference counterpart: device addresses of the model's storage, for harnesses that fill the
 * paged cache directly (any of the outputs may be NULL).  Layers [num_hidden_layers,
 * num_hidden_layers + drafter num_layers) are the drafter's own caches. */
int cpmcu_model_pointers(int layer, uint64_t* k_pool, uint64_t* v_pool, uint64_t* block_table, int* num_pages);

/* No reference counterpart: the library's own stream (a hipStream_t as an integer; created on first use), for
 * harnesses that record events on it or order their own streams against it.  0 if it cannot be created. */
uint64_t cpmcu_stream(void);
/* Synchronise the library's stream.  Also reports (CPMCU_ERR_RUNTIME) an attention launch since the last check whose
 * device-side KV length lay outside what its call had promised -- above max_kv_len / padded_length, or shorter than
 * its rows: such a launch runs on the clamped length (no access leaves the page table) and its output is not valid. */
int cpmcu_synchronize(void);
/* No reference counterpart: merge waits of tree-attention launches that ran out, as counted by the synchronising calls
 * so far (cpmcu_synchronize, cpmcu_verify_and_fix; also printed by cpmcu_print_perf_summary).  A split workgroup that
 * has waited attn_merge_wait_us for the other workgroups of its unit leaves its share of the merge to the last of them
 * and ends: the output is complete, only late.  It happens when the launch's workgroups are not all resident at once,
 * i.e. when another launch holds CUs.  After the first such wait is seen, the device's workspaces go back to the
 * separate merge launch; cpmcu_set_option("attn_merge_in_launch", 1) lets them merge inside the launch again. */
long cpmcu_attention_abandoned_waits(void);
/* Free everything the global model owns (the reference never frees). */
int cpmcu_shutdown(void);

/* ------------------------------------------------------------------------- */
/* 2. Operator-level entry points                                             */
/* ------------------------------------------------------------------------- */

/* KV append -- copy_to_kvcache, src/model/attn.cuh:14-21,42-47,200.
 * Writes T new token rows of one layer into the paged pools at token positions
 * [*kv_len - T, *kv_len).  k_new, v_new: [T][Hkv][128] fp16 row-major.
 * kv_len: device int32[1], total length after the append. */
int cpmcu_kv_append(void* k_pool, void* v_pool, const int32_t* block_table, const void* k_new,
                    const void* v_new, const int32_t* kv_len, int T, int Hkv, void* stream);

/* Bytes of scratch cpmcu_tree_attention needs for these shapes (split-KV partials). */
size_t cpmcu_tree_attention_workspace_bytes(int T, int Hq, int Hkv, int max_kv_len);

/* Tree-verify attention -- mha_fwd_kvcache with a 2-D tree mask,
 * src/flash_attn/flash_api.hpp:292-392; kernel body
 * src/flash_attn/src/flash_fwd_kernel.h:1175-1766; mask src/flash_attn/src/mask.h:139-229;
 * split merge src/flash_attn/src/flash_fwd_kernel.h:2320-2501.
 *   q   [T][Hq][128] fp16;  out [T][Hq][128] fp16
 *   kv_len: device int32[1] = P + T (the true length is read on the device, as
 *           the reference reads cu_seqlens_k, flash_api.hpp:383-385); the tree
 *           nodes are the last T tokens, in node order.
 *   max_kv_len: host upper bound of *kv_len used for the launch geometry and the
 *           split partition (the reference's padded_length); keep it tight (within
 *           a few hundred tokens of *kv_len).  block_table must have an entry for
 *           every page below ceil(max_kv_len / 256).
 *   k_new, v_new: [T][Hkv][128] fp16 rows of the T tree nodes, or both NULL.  When
 *           given, the kernel performs the KV append of src/model/attn.cuh:14-21,200
 *           itself: the rows are used for positions [*kv_len - T, *kv_len) and are
 *           written into the pools, so no separate cpmcu_kv_append call is needed.
 *           When NULL the rows must already be in the cache.
 *   mask [T][mask_words] uint64, mask_k_range: bit j of row i = query i attends the key at
 *           position *kv_len - mask_k_range + j; keys before that are all visible, and the
 *           causal bound (query i sees keys up to its own position *kv_len - T + i) applies
 *           as well (src/flash_attn/src/mask.h:185-203).  mask_k_range = T (or 0, which means
 *           T) is the verify tree (bit j = tree node j); mask_k_range = k * d > T is the
 *           drafter's own attention over its previous d - 1 rounds of k draft tokens
 *           (Mask(eagle_mask_2d, k, k * d), src/model/minicpm4/minicpm4_eagle.cuh:359).
 *           mask = NULL: causal chain.  mask_words = ceil(mask_k_range / 64).
 *   scale: softmax scale (1/sqrt(128) in the reference, flash_api.hpp:360).
 *   workspace: device scratch of at least ..._workspace_bytes(), may be NULL
 *           when that is 0.  Calls that may overlap on one GPU must use different
 *           workspaces: the split partials live there, and the library keys the
 *           arrival counters of the in-launch merge by this pointer (a launch with at
 *           most 32 splits and at most one workgroup per CU merges its own partials;
 *           its workgroups wait for each other, which needs them all resident -- see
 *           "attn_merge_in_launch" above).
 *   num_splits_override: 0 = choose from max_kv_len; >0 forces the KV split count.
 * max_kv_len is limited to 2^30. */
int cpmcu_tree_attention(const void* q, void* k_pool, void* v_pool, const int32_t* block_table,
                         const int32_t* kv_len, int max_kv_len, const void* k_new, const void* v_new,
                         const uint64_t* mask, int mask_words, int mask_k_range, int T, int Hq, int Hkv, float scale,
                         void* out,
                         void* workspace, size_t workspace_bytes, int num_splits_override, void* stream);

/* No reference counterpart: whether launches on this workspace merge their split partials themselves (1) or leave it
 * to the separate merge launch (0).  The library keeps a block of arrival counters per workspace pointer it has met on a
 * device (32 per device, kept until the library's own workspace is freed at cpmcu_shutdown; further workspaces get
 * none), and takes every workspace of a device off the in-launch merge once a merge wait has been abandoned there
 * (see cpmcu_attention_abandoned_waits).  Asking assigns a block to a workspace that has none yet. */
int cpmcu_tree_attention_merge_mode(const void* workspace);
/* No reference counterpart: tells the library that an attention workspace is about to be freed, so that its block of
 * arrival counters can go to another workspace.  None of its launches may be in flight, and no captured graph that holds
 * one may be replayed afterwards.  A workspace the library has never met is ignored. */
int cpmcu_tree_attention_release_workspace(const void* workspace);

/* No reference counterpart: which kernels a cpmcu_tree_attention* call of this shape launches, without
 * launching -- for reports that must name the instantiation actually taken.  kernel_names receives e.g.
 * "tree_attn_split_kernel<2,false>+tree_attn_combine_kernel" (beyond 32 splits: "+tree_attn_combine_wide_kernel"); the
 * outputs may each be NULL. */
int cpmcu_tree_attention_plan(int T, int Hq, int Hkv, int max_kv_len, int with_rope, int block_window_size,
                              int num_splits_override, char* kernel_names, size_t kernel_names_bytes, int* num_splits,
                              int* kv_groups, int* num_workgroups);

/* Rotary embedding of the T tree rows -- RotaryEmbedding::prefill / rotary_embedding_kernel,
 * src/model/rotary.cuh:7-34,61-63, which Attention::decode runs on q and k before the append
 * (src/model/attn.cuh:199-200).  The angles depend on (position, frequency) only, so they are computed
 * once per step, not once per layer and element:
 *   cos_sin [T][64][2] fp32 = (cos, sin)(float(position_ids[t]) * inv_freq[col])       cpmcu_rope_table
 * and applied either inside the attention kernel (cpmcu_tree_attention_rope: the queries rotate in
 * registers as they are loaded, the appended K rows rotate in the LDS tile on their way into the pool;
 * q and k_new themselves are not modified; without k_new only q rotates) or in place by
 * cpmcu_rope_apply (q [T][Hq][128], k [T][Hkv][128]), the reference's own form.  Pair (d, d + 64):
 *   x'[d] = f16(x[d] * cos - x[d+64] * sin),  x'[d+64] = f16(x[d] * sin + x[d+64] * cos)   (fp32 arithmetic). */
int cpmcu_rope_table(const int32_t* position_ids, const float* inv_freq, int T, float* cos_sin, void* stream);
int cpmcu_rope_apply(const float* cos_sin, int T, int Hq, int Hkv, void* q, void* k, void* stream);
int cpmcu_tree_attention_rope(const void* q, void* k_pool, void* v_pool, const int32_t* block_table,
                              const int32_t* kv_len, int max_kv_len, const void* k_new, const void* v_new,
                              const float* rope_cos_sin, const uint64_t* mask, int mask_words, int mask_k_range,
                              int T, int Hq, int Hkv, float scale, void* out,
                              void* workspace, size_t workspace_bytes, int num_splits_override, void* stream);

/* The same attention with the block-granular sliding window of the drafter's own layer --
 * fwdIterator without a block mask, src/flash_attn/src/flash_blockmask.h:9,16,32,43-46, reached through
 * mha_fwd_kvcache's block_window_size (src/flash_attn/flash_api.hpp:316,368) = Attention::window_size
 * (src/model/attn.cuh:228) = eagle_window_size of init_minicpm4_eagle_model.
 *   block_window_size: in tokens; 0 = no window, otherwise >= 128.  With P = *kv_len - T, the key
 *           blocks of 128 below  ceil(P / 128) - block_window_size / 128  are not visited (the
 *           reference's split-KV kernel walks K in blocks of 128 for head dimension 128,
 *           src/flash_attn/src/flash_fwd_launch_template.h:208): the queries see the keys from
 *           128 * that block index on, under the same mask and causal rules as above.
 *   rope_cos_sin: as for cpmcu_tree_attention_rope, or NULL for inputs that are already rotated.
 * The kernel starts its KV stream at the window's first block, so the cost follows the window, not
 * the context; max_kv_len still bounds *kv_len and the page table.  With more than 64 rows the window start is
 * taken once, from the first row, for all rows; the reference derives it per 64-row block of queries
 * (src/flash_attn/src/flash_blockmask.h:32) but asserts tree_size <= 64, so that case lies beyond it and is not
 * pinned against anything. */
int cpmcu_tree_attention_window(const void* q, void* k_pool, void* v_pool, const int32_t* block_table,
                                const int32_t* kv_len, int max_kv_len, const void* k_new, const void* v_new,
                                const float* rope_cos_sin, int block_window_size,
                                const uint64_t* mask, int mask_words, int mask_k_range,
                                int T, int Hq, int Hkv, float scale, void* out,
                                void* workspace, size_t workspace_bytes, int num_splits_override, void* stream);

/* remap_copy -- src/model/tree_drafter.cuh:79-86,103-107: dst[r][:] = src[remap[r]][:]. */
int cpmcu_gather_rows(const void* src, const int32_t* remap, int rows, int dim, void* dst, void* stream);

/* Weight layouts of the two head operators (w_layout).
 * CPMCU_W_ROW_MAJOR: [V][H] fp16 as the reference keeps it (src/model/linear.cuh:39-47).
 * CPMCU_W_TILED: the same numbers in MFMA operand order, [ceil(V/16)][H/32][64 lanes][8 halves]
 *   (rows beyond V are zero): a wave's 16-row block is one contiguous stream of H*32 bytes, which
 *   the GPU reads ~20 % faster than 16 strided rows.  Built once at load time by
 *   cpmcu_head_weight_tile.  Logits of the two layouts agree to fp16 rounding of the same fp32
 *   sums taken in a different order (the K-chunking chosen per layout differs). */
#define CPMCU_W_ROW_MAJOR 0
#define CPMCU_W_TILED 1
size_t cpmcu_head_weight_tiled_bytes(int V, int H);
/* w [*][H] fp16 row-major -> w_tiled (cpmcu_head_weight_tiled_bytes(V, H) bytes, must not alias w).
 * Row r of the result is row row_remap[r] of w when row_remap is given (this is remap_copy,
 * src/model/tree_drafter.cuh:79-86, fused with the re-tiling), else row r.  H % 32 == 0. */
int cpmcu_head_weight_tile(const void* w, const int32_t* row_remap, int V, int H, void* w_tiled, void* stream);

/* Bytes of scratch the two head operators need. */
size_t cpmcu_head_workspace_bytes(int n, int V);

/* FR-Spec draft head with fused log-softmax statistics, top-k and id map-back --
 * Linear::prefill (src/model/linear.cuh:8-37,73-79) + log_softmax
 * (src/model/eagle.cuh:29-89) + TopK::prefill (src/model/topk.cuh:158-213,255-288)
 * + remap (src/model/tree_drafter.cuh:88-90).
 *   hidden [n][H] fp16 (n <= 16); w: the gathered sub-matrix, V rows, in layout w_layout;
 *   logits [n][V] fp16 scratch/output (raw logits z);
 *   row_stats [n][2] fp32 output: (max z, ln sum exp(z - max));
 *   topk_val [n][k] fp16 = f16((z - max) - lnsum); topk_pos [n][k] int32 index into w;
 *   topk_ids [n][k] int32 = token_id_remap[topk_pos] (token_id_remap NULL -> ids = pos).
 * Ordering: value descending, ties -> lower index (src/model/topk.cuh:17). k <= 32. */
int cpmcu_frspec_head_topk(const void* hidden, const void* w, int w_layout, const int32_t* token_id_remap, int n, int V,
                           int H, int k, void* logits, float* row_stats, void* topk_val, int32_t* topk_pos,
                           int32_t* topk_ids, void* workspace, size_t workspace_bytes, void* stream);

/* The call above runs as ONE launch when the shape allows it (CPMCU_W_TILED weights, k <= 16, V a multiple of 8 with one
 * or two full passes of 16-row blocks over the GPU -- the FR-Spec vocabulary of 32768 is one) and one of the library's 8
 * publication states per device is free for (workspace, grid size): every GEMM workgroup publishes its k..16 best
 * (value, index, token id) per hidden row as tagged 64-bit words, and the first n workgroups to finish rank one row
 * each.  Same outputs, bit for bit, as the two-launch form (cpmcu_set_option("frspec_fused", 0)); logits are complete
 * when the launch ends.  A state stays with its (workspace, grid) until cpmcu_head_release_workspace; calls that
 * overlap on one GPU must use different workspaces, as before.  A finisher waits at most frspec_wait_us (option,
 * default 50000) for the other workgroups of its launch to become resident; if that runs out its row holds index -1,
 * the next synchronising call of the library returns CPMCU_ERR_RUNTIME, and the device goes back to two launches.
 * No counterpart in the reference, which runs these steps as separate kernels (minicpm4_eagle.cuh:366-372).
 * cpmcu_frspec_head_mode: 1 if a call of this shape on this workspace is one launch (assigns a state if needed), else 0.
 * cpmcu_frspec_fused_rows: rows seen by the library's synchronisations so far -- finished from the published words,
 * redone from the logits in memory (rows dominated by equal values), not finished (wait ran out); pointers may be NULL. */
int cpmcu_frspec_head_mode(const void* workspace, int w_layout, int n, int V, int H, int k);
int cpmcu_head_release_workspace(const void* workspace);
int cpmcu_frspec_fused_rows(long* fused_rows, long* slow_rows, long* timeouts);

/* Target head with fused arg-max -- LMHead::prefill (src/model/linear.cuh:82-101;
 * fp16 pre-scale by head_scale when apply_scale != 0) + torch argmax
 * (cpmcu/speculative/tree_drafter.py:153,233; lowest index on ties).
 *   hidden [n][H] fp16 (n <= 128); w: V rows in layout w_layout; logits [n][V] fp16 or NULL (not
 *   materialised); gt int32[n] or NULL. */
int cpmcu_lm_head_argmax(const void* hidden, const void* w, int w_layout, int n, int V, int H, int apply_scale,
                         float head_scale, void* logits, int32_t* gt, void* workspace,
                         size_t workspace_bytes, void* stream);

/* No reference counterpart: the GEMM kernel a head call of this shape launches (e.g.
 * "head_gemm_chunked_kernel<4,4,256,2>") and its workgroup count, without launching. */
int cpmcu_head_plan(int n, int V, int H, int w_layout, char* kernel_name, size_t kernel_name_bytes, int* num_workgroups);

/* The target head's GEMM without its finishing launch: the per-workgroup arg-max partials stay in
 * `workspace` (same size as for cpmcu_lm_head_argmax) and are finished by cpmcu_verify_tail, which is their
 * only consumer in a verify step.  *num_partials / *partial_stride (host) describe them for that call.
 * logits as above, or NULL. */
int cpmcu_lm_head_partials(const void* hidden, const void* w, int w_layout, int n, int V, int H, int apply_scale,
                           float head_scale, void* logits, void* workspace, size_t workspace_bytes, int* num_partials,
                           int* partial_stride, void* stream);

/* cpmcu_lm_head_argmax for callers that cannot allocate device memory or bring a workspace: code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the
 * reference.  Same arguments and results as cpmcu_lm_head_argmax without the workspace: the per-workgroup
 * arg-max partials live in a device array built into the library
 * (cpmcu_lm_head_argmax_static_scratch_bytes() = 1 MiB, held by every GPU the library runs on until the
 * process ends), which bounds the call to n <= 128 rows; more rows are rejected with
 * CPMCU_ERR_INVALID_ARGUMENT.  The call allocates nothing and synchronises nothing; the first call on a
 * device looks up that device's copy of the array (make it outside a capture).  stream = NULL is HIP's
 * null stream here, not the library's own stream (which is created on first use).
 * All calls on one GPU share the array, so calls that overlap on one GPU (different streams) race;
 * calls on one stream are ordered and need no clearing in between: every launch rewrites the partials
 * it reads. */
size_t cpmcu_lm_head_argmax_static_scratch_bytes(void);
int cpmcu_lm_head_argmax_static(const void* hidden, const void* w, int w_layout, int n, int V, int H, int apply_scale,
                                float head_scale, void* logits, int32_t* gt, void* stream);

/* log_softmax in place -- src/model/eagle.cuh:29-89.  x [n][dim] fp16 (bf16 under the dtype option), any dim, 2-byte
 * alignment is enough; row_stats [n][2] fp32 (max, ln sum) output, may be NULL. */
int cpmcu_log_softmax(void* x, int n, int dim, float* row_stats, void* stream);

/* TopK::prefill -- src/model/topk.cuh:255-288: per row the `top` largest values,
 * value descending, ties -> lower index.  top <= min(dim, 128); any dim and any 2-byte aligned x (rows of whole
 * 16-byte pieces -- dim a multiple of 8, x on 16 bytes -- are read fastest); rows of more than 32768 elements need
 * top x ceil(dim / 32768) <= 1024.  val [n][top] in the element type, pos int32 [n][top].
 * workspace: at least cpmcu_topk_workspace_bytes(n, dim, top) (used for rows of more than 32768 elements). */
size_t cpmcu_topk_workspace_bytes(int n, int dim, int top);
int cpmcu_topk(const void* x, int n, int dim, int top, void* val, int32_t* pos, void* workspace,
               size_t workspace_bytes, void* stream);

/* remap -- src/model/tree_drafter.cuh:88-90: out[i] = token_id_remap[in[i]]. */
int cpmcu_remap(const int32_t* in, int n, const int32_t* token_id_remap, int32_t* out, void* stream);

/* Greedy tree acceptance -- verify_kernel, src/model/tree_drafter.cuh:5-46, extended
 * to T <= 128 (mask_words = ceil(T/64) uint64 per row; tournament over
 * next_pow2(max(64, T)) slots, identical to the reference for T <= 64).
 *   pred int32[T] in: draft ids; out: pred[0..a) = node indices of the accepted
 *   path in depth order (the reference's scatter, :42-45).
 *   best int32[2] out: (a, winning node).  cache_length: device int32[1] = P. */
int cpmcu_tree_accept(int T, int32_t* pred, const int32_t* gt, const int32_t* position_ids,
                      const int32_t* cache_length, const uint64_t* attn_mask, int mask_words,
                      const int32_t* tree_parent, int32_t* best, void* stream);

/* Accepted-path compaction -- fix_kv_cache, src/model/tree_drafter.cuh:48-77,97-101.
 * For every layer l < num_layers and d < a: token P + pred[d] of k_pools[l] /
 * v_pools[l] moves to token P + d; then pred[d] <- gt[pred[d]] (accepted ids).
 * a is read on the device from best[0] (no host round trip); max_accept bounds it
 * for the launch.  k_pools / v_pools: device arrays of num_layers pool pointers. */
int cpmcu_kv_compact(void* const* k_pools, void* const* v_pools, int num_layers, const int32_t* block_table,
                     int Hkv, int32_t* pred, const int32_t* gt, const int32_t* cache_length,
                     const int32_t* best, int max_accept, void* stream);

/* The rest of verify() in the same two launches as cpmcu_kv_compact --
 * MiniCPM4EagleImpl::verify, src/model/minicpm4/minicpm4_eagle.cuh:398-418, and the host side of the
 * loop, cpmcu/speculative/tree_drafter.py:222,243-249.  On top of the compaction and the accepted ids:
 *   prev_hidden[d][:] = hidden[path[d]][:] for d < a   (remap_hidden, src/model/eagle.cuh:108-115,169-172;
 *       hidden [T][hidden_dim] fp16 = the target's final-norm output; both NULL: skipped);
 *   next_position_ids[d] = P + d for d < a             (make_arange, src/model/eagle.cuh:125-127,184-186; NULL: skipped);
 *   result[0] = a, result[1 + d] = accepted id d       (int32[1 + max_accept]; device memory or pinned,
 *       device-visible host memory: one read after one synchronisation replaces the reference's
 *       reads of the accept length and of tree_draft_ids[:a]; NULL: skipped);
 *   CPMCU_COMMIT_ADVANCE_LENGTH: cache_length[0] = P + a on the device (the host's
 *       cache_length[0] = prefix_length + i of the next iteration), and kv_len[0] += a when kv_len is
 *       given: the device scalar P + T that the attention calls read (cpmcu/llm.py:272), so the next
 *       step can be enqueued, or a captured graph of it replayed, without the host knowing a;
 *   CPMCU_COMMIT_NEXT_ROOT: pred[0] = the last accepted id (tree_draft_ids[0] = tree_draft_ids[a - 1]). */
int cpmcu_accept_commit(void* const* k_pools, void* const* v_pools, int num_layers, const int32_t* block_table,
                        int Hkv, int32_t* pred, const int32_t* gt, int32_t* cache_length, int32_t* kv_len,
                        const int32_t* best, int max_accept, const void* hidden, int hidden_dim, void* prev_hidden,
                        int32_t* next_position_ids, int32_t* result, int flags, void* stream);

/* The whole tail of a verify step in ONE launch -- MiniCPM4EagleImpl::verify,
 * src/model/minicpm4/minicpm4_eagle.cuh:398-418: greedy acceptance
 * (src/model/tree_drafter.cuh:5-46), compaction of the accepted rows in every cache (:48-77), the accepted
 * ids (:74-76), the gather of the accepted hidden rows (src/model/eagle.cuh:108-115) and, in front of all
 * that, the finish of the target arg-max when the head leaves it as partials (cpmcu_lm_head_partials).
 * Every workgroup of the launch recomputes the acceptance from the same few hundred bytes and then moves
 * its own cache stream, so nothing waits for a second launch.  Unlike cpmcu_tree_accept / cpmcu_kv_compact
 * the draft ids are read-only and every result has its own array:
 *   draft_ids int32[T] in; gt int32[T] in, or NULL with head_partials = the workspace of
 *   cpmcu_lm_head_partials (+ its num_partials, partial_stride); cache_length int32[1] = P, read only;
 *   hidden [T][hidden_dim] / prev_hidden [T][hidden_dim]: prev_hidden[d] = hidden[path[d]], both NULL to skip;
 *   outputs (each may be NULL): gt_out int32[T]; best int32[2] = (a, winning node); path int32[T] (first a
 *   entries: node indices by depth); accepted_ids int32[T] (first a entries: gt[path[d]]);
 *   next_position_ids int32[T] (P + d); result int32[1 + T] = (a, ids), device or pinned host memory.
 * The in-place updates that other workgroups of that launch must not see are a second, single-workgroup
 * launch, cpmcu_verify_tail_inplace: pred[0..a) <- accepted ids (what the reference's verify leaves in
 * tree_draft_ids; pred may be NULL), and with flags as for cpmcu_accept_commit cache_length[0] += a,
 * kv_len[0] += a (kv_len may be NULL), position_ids[0..T) += a (may be NULL: the positions a tree of the same
 * shape has in the next step), pred[0] <- the last accepted id instead of the id copy. */
int cpmcu_verify_tail(void* const* k_pools, void* const* v_pools, int num_layers, const int32_t* block_table, int Hkv,
                      int T, const int32_t* draft_ids, const int32_t* gt, const void* head_partials, int num_partials,
                      int partial_stride, const int32_t* position_ids, const int32_t* cache_length,
                      const uint64_t* attn_mask, int mask_words, const int32_t* tree_parent, const void* hidden,
                      int hidden_dim, void* prev_hidden, int32_t* gt_out, int32_t* best, int32_t* path,
                      int32_t* accepted_ids, int32_t* next_position_ids, int32_t* result, void* stream);
int cpmcu_verify_tail_inplace(const int32_t* best, const int32_t* accepted_ids, int T, int32_t* pred, int32_t* cache_length,
                              int32_t* kv_len, int32_t* position_ids, int flags, void* stream);

/* ---- Draft-tree construction around the FR-Spec head (the tree bookkeeping of draft()) ----
 * src/model/minicpm4/minicpm4_eagle.cuh:319-393 with src/model/eagle.cuh:91-106,121-127,188-214.
 * k = topk_per_iter (<= 32), num_iter iterations (k * num_iter <= 64: the draft mask is one
 * uint64 per live node, as in the reference).  `state` is a caller-owned device buffer of
 * cpmcu_draft_tree_state_bytes(k, num_iter) bytes that holds tried_history_val / _pos / _parent,
 * eagle_mask_2d and the running log-probs between the calls of one draft.
 *   begin  (d = 0, :319-332): topk_val fp16[k] / topk_pos int32[k] = top-k of the first row's
 *          log-probs.  next_ids int32[k] out: the ids to embed next (mapped through
 *          token_id_remap unless it is NULL).  draft_mask uint64[k] out (may be NULL).
 *   extend (d >= 1, :367-382): topk_val fp16[k][k] (in/out: the row's running log-prob is added,
 *          rounded to fp16 -- cumsum, eagle.cuh:103-106) / topk_pos int32[k][k].  Out: next_ids
 *          [k], parent_rows int32[k] (row of the previous hidden states each new node continues:
 *          remap_hidden's index, may be NULL), draft_mask [k] for the next draft-layer attention.
 *   finish (:385-393): selects the tree_size - 1 best candidates of the history and writes
 *          tree_draft_ids[1..tree_size) (entry 0, the root token, is the caller's),
 *          tree_position_ids [tree_size] (P + depth; P read from the device scalar
 *          cache_length[0] -- the reference copies it to the host first, :305),
 *          tree_attn_mask [tree_size][ceil(tree_size/64)], tree_parent [tree_size].
 * Ordering everywhere: value descending, equal values -> lower index (src/model/topk.cuh:17). */
size_t cpmcu_draft_tree_state_bytes(int k, int num_iter);
int cpmcu_draft_tree_begin(void* state, int k, int num_iter, const void* topk_val, const int32_t* topk_pos,
                           const int32_t* token_id_remap, int32_t* next_ids, uint64_t* draft_mask, void* stream);
int cpmcu_draft_tree_extend(void* state, int k, int num_iter, int d, void* topk_val, const int32_t* topk_pos,
                            const int32_t* token_id_remap, int32_t* next_ids, int32_t* parent_rows,
                            uint64_t* draft_mask, void* stream);
int cpmcu_draft_tree_finish(void* state, int k, int num_iter, int tree_size, const int32_t* cache_length,
                            const int32_t* token_id_remap, int32_t* tree_draft_ids, int32_t* tree_position_ids,
                            uint64_t* tree_attn_mask, int32_t* tree_parent, void* stream);

#ifdef __cplusplus
}
#endif
#endif
