/*
 * CPU oracle for the speculative-decoding verify/draft path of CPM.cu.
 *
 * TEST INFRASTRUCTURE ONLY.  This library is the checker: it is linked or
 * loaded by the tests, by the smoke check and by the CPU-baseline leg of the
 * benchmark, never by the product path.  It restates, in plain C++ on the
 * host, what the reference computes on this path; every function cites the
 * reference file:line it follows (paths relative to the reference checkout).
 *
 * fp16 values cross this interface as raw uint16_t bit patterns (IEEE
 * binary16).  Products of two halves are exact in fp32; accumulation is fp32
 * in a fixed, documented order, so results are deterministic and independent
 * of the thread count.
 *
 * Parity status: the reference ships no golden vectors, known-answer tests
 * or fixtures for any function on this path, and its CUDA sources cannot be
 * built here (no nvcc, the CUTLASS submodule is empty), so parity with the
 * reference's own bits is unpinned.  What pins each function instead is
 * listed next to it ("pinned by").
 */
#ifndef CPMCU_ORACLE_H
#define CPMCU_ORACLE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- fp16 helpers (round-to-nearest-even) ----
 * pinned by: numpy.float16 conversion on all 65536 half patterns and on
 * random / boundary floats. */
void orc_f16_to_f32(const uint16_t* in, float* out, int64_t n);
void orc_f32_to_f16(const float* in, uint16_t* out, int64_t n);

/* ---- element type ----
 * Every 16-bit tensor of the functions below is IEEE binary16 by default; orc_set_dtype(1) makes it bfloat16 for the
 * calls that follow (0 switches back): the reference builds its templates for both (src/entry.cu:26-59,
 * torch_dtype 0 / 1).  Rounding is to nearest even in both; sums stay fp32.
 * pinned by: torch's CPU bfloat16 conversion on all 65536 patterns and on random / boundary floats. */
void orc_set_dtype(int dtype);
int orc_get_dtype(void);
void orc_bf16_to_f32(const uint16_t* in, float* out, int64_t n);
void orc_f32_to_bf16(const float* in, uint16_t* out, int64_t n);

/* Number of worker threads the threaded entry points will use. */
int orc_num_threads(void);
void orc_set_num_threads(int n);

/* ---- A1: tree-verify attention (one layer) ----
 * Follows src/flash_attn/flash_api.hpp:292-392 (launcher: layouts, scale),
 * src/flash_attn/src/mask.h:139-229 (tree bit + causal mask of the last
 * mask_k_range columns), src/flash_attn/src/softmax.h:66-91,239-256
 * (exp2 with scale*log2e, normalisation by the row sum),
 * src/flash_attn/src/flash_fwd_kernel.h:1266 (kv head = q head / group),
 * :1610-1615 (P rounded to fp16 before P.V), src/model/attn.cuh:14-21
 * (tree K/V rows already appended at cache rows [P, P+T)).
 *
 *   q    [T][Hq][D]          fp16
 *   k,v  [P+T][Hkv][D]       fp16, flat logical caches (row = token)
 *   mask [T][mask_words]     bit j of row i (word j/64, bit j%64): query i
 *                            attends the key at column P + T - mask_k_range + j
 *                            (mask_k_range >= T trailing columns are governed
 *                            by the mask; = T for the verify tree, = k*d for
 *                            the draft layers, minicpm4_eagle.cuh:359).  The
 *                            causal bound column <= P + i is applied as well
 *                            (mask.h:185-186,207-211).
 *   out  [T][Hq][D]          fp16
 *   lse  [T][Hq]             fp32 or NULL: max*scale + ln(sum)
 * One global row max (no blocking); the blocked/split evaluation of the
 * reference differs only in which max each p is taken against.
 * pinned by: fp64 closed-form softmax attention (numpy), torch CPU
 * scaled_dot_product_attention for chain trees / boolean masks, root-only
 * tree == one-token decode, non-ancestor perturbation invariance, GQA group
 * mapping. */
void orc_tree_attention(const uint16_t* q, const uint16_t* k, const uint16_t* v,
                        const uint64_t* mask, int T, int P, int Hq, int Hkv, int D,
                        int mask_words, int mask_k_range, float scale, uint16_t* out, float* lse);

/* The same with the block-granular sliding window of the drafter's own layer
 * (src/flash_attn/src/flash_blockmask.h:9,16,32,43-46; kBlockN = 128 for head
 * dimension 128, src/flash_attn/src/flash_fwd_launch_template.h:208; the value is
 * Attention::window_size, src/model/attn.cuh:228 = eagle_window_size):
 * with block_window_size > 0 the key blocks of 128 below
 *   k_window_left = ceil(P / 128) - block_window_size / 128
 * are skipped whole; 0 = no window.
 * pinned by: equality with orc_tree_attention on the cache cut to its visible
 * keys [128 * k_window_left, P + T), identity for windows that cover the whole
 * context, fp64 closed form with the explicit visible set. */
void orc_tree_attention_window(const uint16_t* q, const uint16_t* k, const uint16_t* v,
                               const uint64_t* mask, int T, int P, int Hq, int Hkv, int D,
                               int mask_words, int mask_k_range, int block_window_size, float scale,
                               uint16_t* out, float* lse);

/* ---- a7: load-time gather of the frequency-ranked rows ----
 * src/model/tree_drafter.cuh:79-86,103-107:  dst[r][:] = src[remap[r]][:].
 * pinned by: numpy fancy indexing. */
void orc_gather_rows(const uint16_t* src, const int32_t* remap, int rows, int dim, uint16_t* dst);

/* ---- a6 / a11: lm_head GEMM ----
 * src/model/linear.cuh:8-37 (out = in . W^T, fp32 accumulate, fp16 out) and
 * :82-101 (LMHead: hidden pre-scaled by head_scale in fp16 when
 * apply_scale != 0; src/model/elementwise.cuh:34-41).
 *   hid [n][H], w [V][H] -> logits [n][V] fp16.
 * Accumulation order: 16 interleaved partial sums over k (k mod 16), then a
 * fixed pairwise tree.  cuBLAS's order is unknown, so logits are
 * tolerance-level against any GPU.
 * pinned by: fp64 dot products (numpy) within fp16 rounding. */
void orc_lm_head(const uint16_t* hid, const uint16_t* w, int n, int V, int H,
                 int apply_scale, float head_scale, uint16_t* logits);

/* ---- a8: log-softmax in place ----
 * src/model/eagle.cuh:29-89:  m = max x; s = sum expf(x - m) (fp32);
 * x <- f16((x - m) - logf(s)).  Sum order: ascending index.
 * m_out / lse_out (per row, fp32, lse_out = logf(s)) may be NULL.
 * pinned by: fp64 log-softmax (scipy.special.log_softmax) within one fp16
 * ulp; exact on rows where s is a power of two. */
void orc_log_softmax(uint16_t* x, int n, int dim, float* m_out, float* lse_out);

/* Staged variant: applies  x <- f16((x - m[r]) - lse[r])  with row statistics
 * supplied by the caller (e.g. read back from the device), so that top-k ids
 * can be compared bit-exactly although expf/logf and the sum order differ. */
void orc_log_softmax_apply(uint16_t* x, int n, int dim, const float* m, const float* lse);

/* ---- a9: top-k, value descending, ties -> lower index first ----
 * src/model/topk.cuh:6-69 (comparator :17, merge :26,37), :158-213, :255-288.
 * -inf is an ordinary value; top may exceed 32 (the reference's re-masking
 * passes produce the same sorted prefix).  Requires top <= dim.
 *   x [n][dim] fp16 -> val [n][top] fp16, pos [n][top] int32.
 * pinned by: numpy lexsort on (index, -value) incl. heavy ties and -inf. */
void orc_topk(const uint16_t* x, int n, int dim, int top, uint16_t* val, int32_t* pos);

/* ---- a10: FR-Spec index -> full-vocabulary id ----
 * src/model/tree_drafter.cuh:88-90: out[i] = remap[in[i]]. */
void orc_remap(const int32_t* in, int n, const int32_t* remap, int32_t* out);

/* ---- a12: arg-max per row, lowest index on ties ----
 * cpmcu/speculative/tree_drafter.py:153,233 (torch argmax on fp16 logits).
 * pinned by: numpy argmax (first occurrence) incl. planted ties. */
void orc_argmax(const uint16_t* logits, int n, int V, int32_t* gt);

/* ---- a13: greedy tree acceptance ----
 * src/model/tree_drafter.cuh:5-46, generalised to T <= 128 with
 * mask_words = ceil(T/64) words per row and a tournament over
 * S = next_pow2(max(64, T)) slots (identical to the reference for T <= 64).
 *   pred [T] draft ids; gt [T] target arg-max per node; pos [T] position ids;
 *   P prefix length; mask [T][mask_words]; parent [T].
 * Outputs: best[0] = accept length a, best[1] = winning node;
 *          path[0..a) = node indices of the accepted path in depth order
 *          (what the reference scatters into pred, :42-45).
 * Returns a.
 * pinned by: brute-force enumeration of root paths on small trees, chain
 * tree == sequential longest-prefix match, a = 1 + depth of deepest fully
 * matched node. */
int orc_tree_accept(int T, int mask_words, const int32_t* pred, const int32_t* gt,
                    const int32_t* pos, int P, const uint64_t* mask, const int32_t* parent,
                    int32_t* best, int32_t* path);

/* ---- a14: accepted-path compaction on flat logical caches ----
 * src/model/tree_drafter.cuh:48-77,97-101: for every cache c and d < a:
 * tmp[d] = cache_c[P + path[d]], then cache_c[P + d] = tmp[d]; finally
 * ids_out[d] = gt[path[d]].
 *   caches: num_caches pointers to [rows][row_halves] fp16.
 * pinned by: numpy fancy-index copy; overlap case path=[0,2,3]. */
void orc_kv_compact(uint16_t* const* caches, int num_caches, int row_halves, int P, int a,
                    const int32_t* path, const int32_t* gt, int32_t* ids_out);
void orc_rope(int T, int Hq, int Hkv, int half_dim, const float* inv_freq, const int32_t* pos, const float* table,
              uint16_t* q, uint16_t* k);
void orc_accept_commit(uint16_t* const* caches, int num_caches, int row_halves, int P, int a, const int32_t* path,
                       const int32_t* gt, const uint16_t* hidden, int hidden_dim, uint16_t* prev_hidden,
                       int32_t* next_pos, int32_t* result, int32_t* new_length, int32_t* next_root);

/* ---- f1: draft-tree construction around the FR-Spec head ----
 * src/model/minicpm4/minicpm4_eagle.cuh:319-393 (the tree bookkeeping of draft()), with
 * src/model/eagle.cuh:91-101 (init_tree, set_parent, update_tree), :103-106 (cumsum),
 * :121-127 (remap_id), :188-214 (build_dynamic_tree).  k = topk_per_iter.
 * State arrays (caller-owned): tried_val/tried_pos [k + (num_iter-1) k^2], tried_parent
 * [k (num_iter-1)], cum [k] (running log-prob of the k live nodes), mask [k] (eagle_mask_2d).
 *   begin : d = 0 (:319-332).  val/pos [k] = top-k of the first row's log-probs.
 *   extend: d >= 1 (:367-382).  val [k][k] (modified: += cum of its row, rounded to fp16),
 *           pos [k][k]; outputs next_ids [k], parent_rows [k] (= selected / k, the row gather
 *           of remap_hidden :376), updated cum, mask, tried_*.
 *   finish: (:385-393) top-(T-1) of tried_val, build_dynamic_tree with pos_offset = P,
 *           ids_out[1..T) = (remap of) tried_pos[selected]; ids_out[0] is left alone.
 *           mask_words = ceil(T/64) words per mask row (the reference has one).
 *           A selected node whose parent was not selected gets parent 0 (the reference reads an
 *           uninitialised slot there; it cannot happen while log-probs are <= 0).
 * token_id_remap may be NULL (frspec_vocab_size == vocab_size, :327-329,:378-382,:389-393).
 * pinned by: an independent reconstruction with explicit node records (ancestor sets by
 * walking parents, depths, exact cumulative sums on dyadic inputs), hand-worked 2-iteration
 * case; parity with the reference's bits unpinned. */
void orc_draft_tree_begin(int k, const uint16_t* val, const int32_t* pos, const int32_t* token_id_remap,
                          uint16_t* tried_val, int32_t* tried_pos, uint16_t* cum, uint64_t* mask, int32_t* next_ids);
void orc_draft_tree_extend(int k, int d, uint16_t* val, const int32_t* pos, const int32_t* token_id_remap,
                           uint16_t* tried_val, int32_t* tried_pos, int32_t* tried_parent, uint16_t* cum,
                           uint64_t* mask, int32_t* next_ids, int32_t* parent_rows);
void orc_draft_tree_finish(int k, int num_iter, int T, int P, const int32_t* token_id_remap,
                           const uint16_t* tried_val, const int32_t* tried_pos, const int32_t* tried_parent,
                           int32_t* ids_out, int32_t* tree_pos, uint64_t* tree_mask, int32_t* tree_parent);

#ifdef __cplusplus
}
#endif
#endif
