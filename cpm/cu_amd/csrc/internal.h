// Declarations shared between the translation units of libcpmcu_amd (not part of the ABI).
#pragma once
#include "common.h"

namespace cpmcu {

// runtime.hip -- kernel-shape switches, read from the environment once when the library is first used
// (CPMCU_ATTN_KV_GROUPS=1|2, CPMCU_HEAD_NO_SHARE) and changed afterwards through cpmcu_set_option.
struct Options {
    int dtype = 0;                 // element type of the 16-bit tensors handed to the operator-level entry points: 0 = fp16,
                                   // 1 = bf16 (process-wide, like the reference's model; cpmcu_init_base_model sets it)
    int attn_kv_groups = 0;        // 0 = chosen per call; 1 / 2 force that tree-attention kernel shape
    int head_share_last_pass = 1;  // 0 keeps the plain row-block mapping of the head GEMM
    int head_stream_kernel = 1;    // 0 keeps tiled weights on the K-chunked kernel (tests compare the two)
    int attn_merge_in_launch = 1;  // 0: the split partials of tree attention are always merged by a launch of their own
    int attn_merge_wait_us = 2000; // longest wait of a workgroup for the others of its merge before it abandons its share
    int frspec_fused = 0;          // 1: the FR-Spec head with its top-k as one launch where the shape allows (measured no faster: off)
    int frspec_wait_us = 50000;    // longest wait of a finisher of the fused FR-Spec launch for the other workgroups' words
    int topk_row_kernel = 1;       // 0: top-k by k rounds per chunk of 2048 elements and a merge launch (tests compare the two)
};
Options& options();

// tree_attention.hip -- two things an attention launch can leave behind for the host: a device-side length outside
// [max(T, mask_k_range), max_kv_len] (the launch worked on the clamped length), and merge waits that ran out.
// attention_report_enqueue copies both words to pinned host memory in stream order (ahead of a synchronisation, never
// under a capture); attention_report_take reads that copy afterwards and clears what it found.
int attention_report_enqueue(hipStream_t st);
int attention_report_take(int* bad_length, unsigned int* abandoned);
void attention_merge_reenable();
// Assigns the counters of the in-launch merge to a workspace on the current device (otherwise done by the first
// launch that uses it outside a stream capture); they stay with it until it is released.
void attention_prepare_workspace(const void* workspace, void* stream);
// For a workspace that is about to be freed, with none of its launches in flight or captured.
void attention_release_workspace(const void* workspace);

// lm_head.hip -- the streaming GEMM with its two epilogues.
constexpr int kHeadModeStats = 0;
constexpr int kHeadModeArgmax = 1;
// The streaming kernel <NB, FP, KC> (tiled weights, one sweep): NB 16-row blocks of hidden rows, FP full passes, KC-column chunks.
#define CPMCU_HEAD_STREAM_SHAPES(X)                                                                           \
    X(1, 1, 512) X(1, 2, 256) X(1, 3, 256) X(1, 4, 256) X(2, 1, 512) X(2, 2, 256) X(2, 3, 256) X(2, 4, 128) \
    X(4, 1, 256) X(4, 2, 256) X(4, 3, 128) X(4, 4, 128) X(8, 1, 128) X(8, 2, 128)
// (row-walking kernel by row blocks of hidden, the K-chunked kernel <NB, NP, KC, NBUF>, or the streaming kernel)
enum class HeadShape { Row1, Row2, Row4, Row8, C_1_2_512_2, C_1_4_256_2, C_2_4_256_4, C_2_4_256_2, C_4_4_256_4, C_4_4_256_2, C_8_4_128_2,
                       C_2_4_512_2, C_4_4_128_4, C_8_2_128_2,
#define CPMCU_X(nb, fp, kc) S_##nb##_##fp##_##kc,
                       CPMCU_HEAD_STREAM_SHAPES(CPMCU_X)
#undef CPMCU_X
};
const char* head_shape_name(HeadShape s);
// dry_run: only choose the kernel shape and grid (reported through shape_out / grid_out), launch nothing.
int launch_head_gemm(const void* hidden, const void* w, int w_layout, int n, int V, int H, int apply_scale, float head_scale,
                     int mode, void* logits, float* part_a, float* part_b, int* grid_out, int* stride_out,
                     hipStream_t st, HeadShape* shape_out = nullptr, bool dry_run = false);
int head_max_grid();
// The FR-Spec head with its log-softmax, top-k and id map-back in one launch, when the shape allows it and one of the
// library's publication states is free for (workspace, grid); *launched = false: the caller runs the two launches.
int launch_frspec_fused(const void* hidden, const void* w, int w_layout, const int32_t* token_id_remap, int n, int V, int H, int k,
                        void* logits, float* row_stats, void* topk_val, int32_t* topk_pos, int32_t* topk_ids, const void* workspace,
                        hipStream_t st, bool* launched, bool dry_run = false);
void head_fuse_release_workspace(const void* workspace);
// What fused launches left behind: finishers whose wait ran out (their rows hold -1 / NaN and the call has failed), rows
// redone from the logits in memory, rows finished from the published candidates.  enqueue: copy to pinned host memory
// in stream order; take: read that copy after the synchronisation and clear what was found.
int head_fuse_report_enqueue(hipStream_t st);
int head_fuse_report_take(unsigned int* timeouts, unsigned int* slow_rows, unsigned int* fused_rows);
void head_fuse_reenable();

// topk.hip -- exact top-k (value descending, ties -> lower index) with an optional fused
// log-softmax transform whose row statistics come from the GEMM's per-workgroup partials.
struct TopkStatsSource {
    const float* part_max;  // [grid][stride] or null: rank the raw values
    const float* part_sum;
    int grid, stride;
    float* row_stats;       // [n][2] out: (max, ln sum)
};
int launch_topk(const void* x, int n, int dim, int top, void* val, int32_t* pos, int32_t* ids,
                const int32_t* token_id_remap, const TopkStatsSource* stats, void* workspace,
                size_t workspace_bytes, hipStream_t st);

}  // namespace cpmcu
