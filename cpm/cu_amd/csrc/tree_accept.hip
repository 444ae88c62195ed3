// Greedy tree acceptance, accepted-path KV compaction and KV append on the paged cache (gfx950).
//
// These are byte/integer paths, bound by launch latency (acceptance) and HBM/L2 (compaction moves
// a * 2L * Hkv * 256 bytes): no matrix cores, just coalesced 16-byte row moves for K and strided
// 2-byte moves for the transposed V pages.  The accept length never visits the host between the
// three kernels: compaction reads it from device memory.
#include "common.h"
#include "internal.h"
#include "topk_keys.h"

namespace cpmcu {
namespace {

// verify_kernel, src/model/tree_drafter.cuh:5-46, for T <= 128 (W mask words per row).
__global__ __launch_bounds__(128) void tree_accept_kernel(int T, int W, int32_t* pred, const int32_t* gt,
                                                          const int32_t* pos, const int32_t* cache_length,
                                                          const uint64_t* mask, const int32_t* parent,
                                                          int32_t* best) {
    __shared__ uint64_t s_correct[2];
    __shared__ uint32_t s_best[2];
    const int i = threadIdx.x;
    // :9-20  correct bit i <=> i == 0 or pred[i] == gt[parent[i]]
    const bool ok = (i == 0) || (i < T && pred[i] == gt[parent[i]]);
    const uint64_t ballot = __ballot(ok);
    if ((i & 63) == 0) s_correct[i >> 6] = ballot;
    __syncthreads();
    const int P = cache_length[0];
    // :22-28  a node counts iff every ancestor (its mask row) is correct
    bool full = i < T;
    if (full) {
        for (int w = 0; w < W; ++w) {
            const uint64_t mw = mask[(size_t)i * W + w];
            if ((s_correct[w] & mw) != mw) full = false;
        }
    }
    // :30-36  the tournament folds the slots in halves and the upper slot wins only when strictly
    // greater, so two nodes of equal length meet in the round of their lowest differing index bit and
    // the one with that bit clear wins: a maximum over (accepted length, bit-reversed node index
    // ascending).  One key per node, reduced per wave on the DPP path and across the two waves through
    // LDS.  A node that does not count enters as (1, node 0), the root's entry.
    const uint32_t key = full ? ((uint32_t)(pos[i] - P + 1) << 8) | (255u - (__brev((uint32_t)i) >> 24)) : (1u << 8) | 255u;
    const uint32_t wkey = wave_reduce_b32(key, [](uint32_t a, uint32_t b) { return a > b ? a : b; });
    if ((i & 63) == 0) s_best[i >> 6] = wkey;
    __syncthreads();
    const uint32_t bkey = s_best[0] > s_best[1] ? s_best[0] : s_best[1];
    const int p = (int)(__brev(255u - (bkey & 255u)) >> 24);
    if (i == 0) {
        best[0] = (int32_t)(bkey >> 8);
        best[1] = p;
    }
    // :42-45  scatter the accepted path (node indices by depth) into pred
    // (a node whose position does not lie in [P, P + T) -- positions that were not advanced with the prefix
    // length -- scatters nothing instead of writing outside pred)
    if (i < T && ((mask[(size_t)p * W + (i >> 6)] >> (i & 63)) & 1ull) && (unsigned)(pos[i] - P) < (unsigned)T) pred[pos[i] - P] = i;
}

struct CompactParams {
    void* const* k_pools;
    void* const* v_pools;
    const int32_t* block_table;
    int Hkv;
    const int32_t* pred;  // path: node indices by depth
    const int32_t* cache_length;
    const int32_t* best;
    int max_accept;
    // accepted hidden rows (remap_hidden): extra workgroups behind the num_cache_blocks cache streams
    int num_cache_blocks;
    const f16x8* hidden;
    f16x8* prev_hidden;
    int hidden_pieces;  // 16-byte pieces per hidden row
};

// fix_kvcache_kernel_1/2, src/model/tree_drafter.cuh:48-77, on the paged layout.  One workgroup per
// (layer, K|V, kv head).  Sources are read into registers before any destination of the same batch
// is written; batches go in depth order, and because path[d] >= d a later batch never reads a row
// an earlier batch wrote -- so the reference's staging buffer is not needed.
__global__ __launch_bounds__(256) void kv_compact_kernel(CompactParams p) {
    if ((int)blockIdx.x >= p.num_cache_blocks) {
        // remap_hidden, src/model/eagle.cuh:108-115 (scale 1): prev_hidden[d] = hidden[path[d]], one row per
        // workgroup; the path is still in pred because the ids replace it in a later launch
        const int d = blockIdx.x - p.num_cache_blocks;
        int a = p.best[0];
        a = a < p.max_accept ? a : p.max_accept;
        if (d >= a) return;
        const f16x8* src = p.hidden + (size_t)p.pred[d] * p.hidden_pieces;
        f16x8* dst = p.prev_hidden + (size_t)d * p.hidden_pieces;
        for (int i = threadIdx.x; i < p.hidden_pieces; i += 256) dst[i] = src[i];
        return;
    }
    const int g = blockIdx.x % p.Hkv;
    const int kv = (blockIdx.x / p.Hkv) & 1;
    const int layer = blockIdx.x / (2 * p.Hkv);
    const int tid = threadIdx.x;
    int a = p.best[0];
    a = a < p.max_accept ? a : p.max_accept;
    const int P = p.cache_length[0];
    if (kv == 0) {
        f16* pool = (f16*)p.k_pools[layer];
        const int rr = tid >> 4, ch = tid & 15;  // 16 rows x 16 pieces of 16 bytes
        for (int d0 = 0; d0 < a; d0 += 16) {
            const int d = d0 + rr;
            f16x8 x;
            const bool act = d < a;
            if (act) {
                const int ts = P + p.pred[d];
                const int pg = p.block_table[ts / kPage];
                x = *reinterpret_cast<const f16x8*>(pool + (((size_t)pg * p.Hkv + g) * kPage + ts % kPage) * kHeadDim + ch * 8);
            }
            // the loads above must have returned before any wave overwrites a source row
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __syncthreads();
            if (act) {
                const int td = P + d;
                const int pg = p.block_table[td / kPage];
                *reinterpret_cast<f16x8*>(pool + (((size_t)pg * p.Hkv + g) * kPage + td % kPage) * kHeadDim + ch * 8) = x;
            }
        }
    } else {
        f16* pool = (f16*)p.v_pools[layer];
        const int rr = tid >> 7, dd = tid & 127;  // 2 tokens x 128 dims
        for (int d0 = 0; d0 < a; d0 += 2) {
            const int d = d0 + rr;
            f16 x = (f16)0.f;
            const bool act = d < a;
            if (act) {
                const int ts = P + p.pred[d];
                const int pg = p.block_table[ts / kPage];
                x = pool[(((size_t)pg * p.Hkv + g) * kHeadDim + dd) * kPage + v_slot16(ts % kPage)];
            }
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __syncthreads();
            if (act) {
                const int td = P + d;
                const int pg = p.block_table[td / kPage];
                pool[(((size_t)pg * p.Hkv + g) * kHeadDim + dd) * kPage + v_slot16(td % kPage)] = x;
            }
        }
    }
}

// src/model/tree_drafter.cuh:74-76: pred[d] <- gt[pred[d]] once every cache has been moved -- plus, for
// the one-call form of verify(), what the reference does on the host or in one-line kernels after it
// (src/model/minicpm4/minicpm4_eagle.cuh:411, cpmcu/speculative/tree_drafter.py:222,247-249):
//   next_position_ids[d] = P + d (make_arange, src/model/eagle.cuh:125-127,184-186), result = (a, ids),
//   cache_length += a (and the P + T scalar of the attention calls with it), pred[0] = last accepted id
//   (the next tree's root).
__global__ __launch_bounds__(128) void accepted_ids_kernel(int32_t* pred, const int32_t* gt, const int32_t* best, int max_accept,
                                                           int32_t* cache_length, int32_t* kv_len, int32_t* next_position_ids,
                                                           int32_t* result, int flags) {
    int a = best[0];
    a = a < max_accept ? a : max_accept;
    const int d = threadIdx.x;
    const int P = cache_length ? cache_length[0] : 0;
    int id = 0;
    if (d < a) id = gt[pred[d]];
    __syncthreads();
    if (d < a) {
        pred[d] = id;
        if (next_position_ids) next_position_ids[d] = P + d;
        if (result) result[1 + d] = id;
    }
    if (d == 0) {
        if (result) result[0] = a;
        if (flags & CPMCU_COMMIT_ADVANCE_LENGTH) {
            cache_length[0] = P + a;
            if (kv_len) kv_len[0] += a;
        }
    }
    if (flags & CPMCU_COMMIT_NEXT_ROOT) {
        __syncthreads();
        if (d == a - 1) pred[0] = id;
    }
}

// ---- the whole tail of verify() in one launch ----
// Arg-max finish (when the target head hands over its per-workgroup partials instead of gt), greedy
// acceptance (verify_kernel, src/model/tree_drafter.cuh:5-46), compaction of every cache
// (fix_kvcache_kernel_1/2, :48-77), the gather of the accepted hidden rows (remap_hidden,
// src/model/eagle.cuh:108-115) and the accepted ids (:74-76) with the host-side bookkeeping of
// cpmcu/speculative/tree_drafter.py:222,243-249.  The acceptance is a few hundred bytes of integer work,
// so EVERY workgroup redoes it (and the arg-max finish in front of it) from the same inputs and then does
// its own share: one cache stream, one hidden row, or -- the last workgroup -- the outputs.  Nothing is
// read that another workgroup of the launch writes: the draft ids come in through `draft` and the path /
// accepted ids go out through separate arrays, and no workgroup writes the lengths.
struct TailParams {
    int T, W;
    const int32_t* draft;         // draft token ids (pred on entry of verify)
    const int32_t* gt;            // target arg-max per node, or null: taken from the head's partials
    const float* part_a;          // [num_partials][partial_stride] best value
    const float* part_b;          // [num_partials][partial_stride] best index (int bits)
    int num_partials, partial_stride;
    const int32_t* pos;
    const int32_t* cache_length;  // P (read only)
    const uint64_t* mask;
    const int32_t* parent;
    // compaction
    void* const* k_pools;
    void* const* v_pools;
    const int32_t* block_table;
    int Hkv;
    int num_cache_blocks;         // num_layers * 2 * Hkv workgroups
    // accepted hidden rows: num_hidden_blocks workgroups behind the cache streams
    const f16x8* hidden;
    f16x8* prev_hidden;
    int hidden_pieces, num_hidden_blocks;
    // outputs, written by the last workgroup (any may be null)
    int32_t* gt_out;              // [T]
    int32_t* best;                // (a, winning node)
    int32_t* path;                // [T]: node indices of the accepted path by depth (first a entries)
    int32_t* ids;                 // [T]: accepted token ids (first a entries)
    int32_t* next_position_ids;   // [T]: P + d
    int32_t* result;              // [1 + T]: (a, ids)
};

__device__ inline uint64_t argmax_key(float value, uint32_t index) {
    const uint32_t bits = (uint32_t)__float_as_int(value + 0.f);  // -0 -> +0: they compare equal
    const uint32_t image = bits ^ ((bits >> 31) ? 0xFFFFFFFFu : 0x80000000u);
    return ((uint64_t)image << 32) | (0xFFFFFFFFu - index);
}

constexpr int kTailThreads = 256;

__global__ __launch_bounds__(kTailThreads) void verify_tail_kernel(TailParams p) {
    __shared__ int32_t s_gt[kMaxTree];
    __shared__ int32_t s_path[kMaxTree];
    __shared__ uint64_t s_mask[kMaxTree][2];
    __shared__ uint64_t s_key[kTailThreads];
    __shared__ uint64_t s_correct[2];
    __shared__ uint32_t s_best[2];
    __shared__ int32_t s_pages[2];
    const int tid = threadIdx.x;
    const int T = p.T, W = p.W;
    const int i = tid;

    // Everything the acceptance reads from memory is requested first, so that it arrives under the arg-max
    // finish: the launch is a chain of memory round trips, and these need not be links of it.
    const int P = p.cache_length[0];
    int my_draft = 0, my_parent = 0, my_pos = 0;
    uint64_t mw[2] = {0, 0};
    if (i < T) {
        my_draft = p.draft[i];
        my_parent = p.parent[i];
        my_pos = p.pos[i];
        mw[0] = p.mask[(size_t)i * W];
        if (W > 1) mw[1] = p.mask[(size_t)i * W + 1];
    }
    // the tree rows [P, P + T) lie in at most two logical pages
    if (tid < 2) s_pages[tid] = p.block_table[P / kPage + tid * ((P + T - 1) / kPage > P / kPage ? 1 : 0)];

    // ---- target arg-max per node: given, or the finish of the head's per-workgroup partials (largest value,
    // lowest index among equals: the same 64-bit keys as the head's own finish kernel) ----
    if (p.gt != nullptr) {
        if (tid < T) s_gt[tid] = p.gt[tid];
    } else {
        const int rows = p.partial_stride;        // 16 .. 128, a power of two
        const int row = tid & (rows - 1);
        const int clanes = kTailThreads / rows;   // partial lanes per row
        uint64_t bestk = 0;
        if (row < T) {
            constexpr int kBatch = 32;  // partials of one row requested together: one round trip per batch
            for (int c0 = tid / rows; c0 < p.num_partials; c0 += clanes * kBatch) {
                float av[kBatch];
                uint32_t bv[kBatch];
#pragma unroll
                for (int u = 0; u < kBatch; ++u) {
                    const int c = min(c0 + u * clanes, p.num_partials - 1);  // clamp: a repeat changes nothing in a maximum
                    av[u] = p.part_a[(size_t)c * rows + row];
                    bv[u] = (uint32_t)__float_as_int(p.part_b[(size_t)c * rows + row]);
                }
#pragma unroll
                for (int u = 0; u < kBatch; ++u) {
                    const uint64_t k = argmax_key(av[u], bv[u]);
                    bestk = k > bestk ? k : bestk;
                }
            }
        }
        s_key[tid] = bestk;
        __syncthreads();
        if (tid < rows && tid < T) {
            uint64_t k = s_key[tid];
            for (int l = 1; l < clanes; ++l) {
                const uint64_t o = s_key[l * rows + tid];
                k = o > k ? o : k;
            }
            s_gt[tid] = (int32_t)(0xFFFFFFFFu - (uint32_t)k);
        }
    }
    if (i < kMaxTree) {
        s_mask[i][0] = mw[0];
        s_mask[i][1] = mw[1];
        s_path[i] = i < T ? i : 0;  // (defined even where stale positions scatter nothing)
    }
    __syncthreads();

    // ---- acceptance (as tree_accept_kernel above, on 128 of the threads) ----
    const bool ok = (i == 0) || (i < T && my_draft == s_gt[my_parent]);
    const uint64_t ballot = __ballot(ok);
    if (i < 128 && (i & 63) == 0) s_correct[i >> 6] = ballot;
    __syncthreads();
    bool full = i < T;
    if (full) {
        for (int w = 0; w < W; ++w)
            if ((s_correct[w] & mw[w]) != mw[w]) full = false;
    }
    const uint32_t key = full ? ((uint32_t)(my_pos - P + 1) << 8) | (255u - (__brev((uint32_t)i) >> 24)) : (1u << 8) | 255u;
    const uint32_t wkey = wave_reduce_b32(key, [](uint32_t a, uint32_t b) { return a > b ? a : b; });
    if (i < 128 && (i & 63) == 0) s_best[i >> 6] = wkey;
    __syncthreads();
    const uint32_t bkey = s_best[0] > s_best[1] ? s_best[0] : s_best[1];
    const int win = (int)(__brev(255u - (bkey & 255u)) >> 24);
    int a = (int)(bkey >> 8);
    a = a < T ? a : T;
    if (i < T && ((s_mask[win][i >> 6] >> (i & 63)) & 1ull) && (unsigned)(my_pos - P) < (unsigned)T) s_path[my_pos - P] = i;
    __syncthreads();
    const int page_lo = P / kPage;
    auto page_of = [&](int token) { return s_pages[token / kPage - page_lo]; };

    const int blk = blockIdx.x;
    if (blk < p.num_cache_blocks) {
        // ---- compaction of one (layer, K|V, kv head) stream: sources of a batch are read before any of its
        // destinations is written, batches go in depth order and path[d] >= d, so no staging buffer ----
        const int g = blk % p.Hkv;
        const int kv = (blk / p.Hkv) & 1;
        const int layer = blk / (2 * p.Hkv);
        if (kv == 0) {
            f16* pool = (f16*)p.k_pools[layer];
            const int rr = tid >> 4, ch = tid & 15;  // 16 rows x 16 pieces of 16 bytes
            for (int d0 = 0; d0 < a; d0 += 16) {
                const int d = d0 + rr;
                f16x8 x;
                const bool act = d < a && s_path[d] != d;  // a row that stays where it is moves nothing
                if (act) {
                    const int ts = P + s_path[d];
                    const int pg = page_of(ts);
                    x = *reinterpret_cast<const f16x8*>(pool + (((size_t)pg * p.Hkv + g) * kPage + ts % kPage) * kHeadDim + ch * 8);
                }
                asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                __syncthreads();
                if (act) {
                    const int td = P + d;
                    const int pg = page_of(td);
                    *reinterpret_cast<f16x8*>(pool + (((size_t)pg * p.Hkv + g) * kPage + td % kPage) * kHeadDim + ch * 8) = x;
                }
            }
        } else {
            f16* pool = (f16*)p.v_pools[layer];
            const int rr = tid >> 7, dd = tid & 127;  // 2 tokens x 128 dims
            for (int d0 = 0; d0 < a; d0 += 2) {
                const int d = d0 + rr;
                f16 x = (f16)0.f;
                const bool act = d < a && s_path[d] != d;
                if (act) {
                    const int ts = P + s_path[d];
                    const int pg = page_of(ts);
                    x = pool[(((size_t)pg * p.Hkv + g) * kHeadDim + dd) * kPage + v_slot16(ts % kPage)];
                }
                asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                __syncthreads();
                if (act) {
                    const int td = P + d;
                    const int pg = page_of(td);
                    pool[(((size_t)pg * p.Hkv + g) * kHeadDim + dd) * kPage + v_slot16(td % kPage)] = x;
                }
            }
        }
        return;
    }
    if (blk < p.num_cache_blocks + p.num_hidden_blocks) {
        // remap_hidden (src/model/eagle.cuh:108-115, scale 1): prev_hidden[d] = hidden[path[d]]
        const int d = blk - p.num_cache_blocks;
        if (d >= a) return;
        const f16x8* src = p.hidden + (size_t)s_path[d] * p.hidden_pieces;
        f16x8* dst = p.prev_hidden + (size_t)d * p.hidden_pieces;
        for (int x = tid; x < p.hidden_pieces; x += kTailThreads) dst[x] = src[x];
        return;
    }
    // ---- the last workgroup: every integer result of the step ----
    if (tid < T) {
        if (p.gt_out) p.gt_out[tid] = s_gt[tid];
        if (tid < a) {
            const int node = s_path[tid];
            const int id = s_gt[node];
            if (p.path) p.path[tid] = node;
            if (p.ids) p.ids[tid] = id;
            if (p.next_position_ids) p.next_position_ids[tid] = P + tid;
            if (p.result) p.result[1 + tid] = id;
        }
    }
    if (tid == 0) {
        if (p.best) {
            p.best[0] = a;
            p.best[1] = win;
        }
        if (p.result) p.result[0] = a;
    }
}

// What must not happen inside the launch above because other workgroups still read the old values: the
// in-place updates.  pred[0..a) <- accepted ids (the reference's verify leaves them there,
// src/model/tree_drafter.cuh:74-76), cache_length / kv_len += a, pred[0] <- last accepted id.
__global__ __launch_bounds__(128) void verify_tail_inplace_kernel(const int32_t* best, const int32_t* ids, int T, int32_t* pred,
                                                                  int32_t* cache_length, int32_t* kv_len, int32_t* position_ids, int flags) {
    int a = best[0];
    a = a < T ? a : T;
    const int d = threadIdx.x;
    if (pred && d < a && !(flags & CPMCU_COMMIT_NEXT_ROOT)) pred[d] = ids[d];
    if (position_ids && (flags & CPMCU_COMMIT_ADVANCE_LENGTH) && d < T) position_ids[d] += a;  // same tree shape, prefix a longer
    if (d == 0) {
        if (flags & CPMCU_COMMIT_ADVANCE_LENGTH) {
            cache_length[0] += a;
            if (kv_len) kv_len[0] += a;
        }
        if (pred && (flags & CPMCU_COMMIT_NEXT_ROOT)) pred[0] = ids[a - 1];
    }
}

// copy_to_kvcache, src/model/attn.cuh:14-21: token t of the T new rows goes to position *kv_len - T + t.
__global__ __launch_bounds__(256) void kv_append_kernel(f16* k_pool, f16* v_pool, const int32_t* block_table,
                                                        const f16* k_new, const f16* v_new,
                                                        const int32_t* kv_len, int T, int Hkv) {
    const int t = blockIdx.x;
    const int tok = kv_len[0] - T + t;
    const int pg = block_table[tok / kPage];
    const int slot = tok % kPage;
    const int row_elems = Hkv * kHeadDim;
    for (int i = threadIdx.x; i < row_elems / 8; i += 256) {  // K: 16-byte pieces
        const int g = i / (kHeadDim / 8), ch = i % (kHeadDim / 8);
        *reinterpret_cast<f16x8*>(k_pool + (((size_t)pg * Hkv + g) * kPage + slot) * kHeadDim + ch * 8) =
            *reinterpret_cast<const f16x8*>(k_new + (size_t)t * row_elems + i * 8);
    }
    for (int i = threadIdx.x; i < row_elems; i += 256) {  // V: transposed, one element per dim
        const int g = i / kHeadDim, dd = i % kHeadDim;
        v_pool[(((size_t)pg * Hkv + g) * kHeadDim + dd) * kPage + v_slot16(slot)] = v_new[(size_t)t * row_elems + i];
    }
}

}  // namespace
}  // namespace cpmcu

using namespace cpmcu;

extern "C" int cpmcu_tree_accept(int T, int32_t* pred, const int32_t* gt, const int32_t* position_ids,
                                 const int32_t* cache_length, const uint64_t* attn_mask, int mask_words,
                                 const int32_t* tree_parent, int32_t* best, void* stream) {
    CPMCU_CHECK_ARG(pred && gt && position_ids && cache_length && attn_mask && tree_parent && best,
                    "tree_accept: null pointer argument");
    CPMCU_CHECK_ARG(T >= 1 && T <= kMaxTree, "tree_accept: tree size %d outside [1, %d]", T, kMaxTree);
    CPMCU_CHECK_ARG(mask_words >= 1 && mask_words <= 2 && mask_words * 64 >= T,
                    "tree_accept: mask_words=%d does not cover T=%d", mask_words, T);
    hipLaunchKernelGGL(tree_accept_kernel, dim3(1), dim3(128), 0, resolve_stream(stream), T, mask_words, pred, gt,
                       position_ids, cache_length, attn_mask, tree_parent, best);
    CPMCU_LAUNCH_CHECK();
    return CPMCU_OK;
}

extern "C" int cpmcu_kv_compact(void* const* k_pools, void* const* v_pools, int num_layers,
                                const int32_t* block_table, int Hkv, int32_t* pred, const int32_t* gt,
                                const int32_t* cache_length, const int32_t* best, int max_accept, void* stream) {
    CPMCU_CHECK_ARG(k_pools && v_pools && block_table && pred && gt && cache_length && best,
                    "kv_compact: null pointer argument");
    CPMCU_CHECK_ARG(num_layers >= 1 && Hkv >= 1, "kv_compact: num_layers=%d Hkv=%d", num_layers, Hkv);
    CPMCU_CHECK_ARG(max_accept >= 1 && max_accept <= kMaxTree, "kv_compact: max_accept=%d outside [1, %d]", max_accept, kMaxTree);
    CompactParams p{k_pools, v_pools, block_table, Hkv, pred, cache_length, best, max_accept, num_layers * 2 * Hkv, nullptr, nullptr, 0};
    hipStream_t st = resolve_stream(stream);
    hipLaunchKernelGGL(kv_compact_kernel, dim3(p.num_cache_blocks), dim3(256), 0, st, p);
    CPMCU_LAUNCH_CHECK();
    hipLaunchKernelGGL(accepted_ids_kernel, dim3(1), dim3(128), 0, st, pred, gt, best, max_accept, (int32_t*)nullptr,
                       (int32_t*)nullptr, (int32_t*)nullptr, (int32_t*)nullptr, 0);
    CPMCU_LAUNCH_CHECK();
    return CPMCU_OK;
}

extern "C" int cpmcu_accept_commit(void* const* k_pools, void* const* v_pools, int num_layers,
                                   const int32_t* block_table, int Hkv, int32_t* pred, const int32_t* gt,
                                   int32_t* cache_length, int32_t* kv_len, const int32_t* best, int max_accept,
                                   const void* hidden, int hidden_dim, void* prev_hidden, int32_t* next_position_ids,
                                   int32_t* result, int flags, void* stream) {
    CPMCU_CHECK_ARG(k_pools && v_pools && block_table && pred && gt && cache_length && best,
                    "accept_commit: null pointer argument");
    CPMCU_CHECK_ARG(num_layers >= 1 && Hkv >= 1, "accept_commit: num_layers=%d Hkv=%d", num_layers, Hkv);
    CPMCU_CHECK_ARG(max_accept >= 1 && max_accept <= kMaxTree, "accept_commit: max_accept=%d outside [1, %d]", max_accept, kMaxTree);
    CPMCU_CHECK_ARG((hidden == nullptr) == (prev_hidden == nullptr), "accept_commit: hidden and prev_hidden go together");
    CPMCU_CHECK_ARG(hidden == nullptr || hidden != prev_hidden, "accept_commit: prev_hidden must not alias hidden");
    CPMCU_CHECK_ARG(!hidden || (hidden_dim >= 8 && hidden_dim % 8 == 0), "accept_commit: hidden_dim=%d must be a positive multiple of 8", hidden_dim);
    CPMCU_CHECK_ARG((flags & ~(CPMCU_COMMIT_ADVANCE_LENGTH | CPMCU_COMMIT_NEXT_ROOT)) == 0, "accept_commit: unknown flags 0x%x", flags);
    CompactParams p{k_pools, v_pools, block_table, Hkv, pred, cache_length, best, max_accept, num_layers * 2 * Hkv,
                    (const f16x8*)hidden, (f16x8*)prev_hidden, hidden ? hidden_dim / 8 : 0};
    hipStream_t st = resolve_stream(stream);
    hipLaunchKernelGGL(kv_compact_kernel, dim3(p.num_cache_blocks + (hidden ? max_accept : 0)), dim3(256), 0, st, p);
    CPMCU_LAUNCH_CHECK();
    hipLaunchKernelGGL(accepted_ids_kernel, dim3(1), dim3(128), 0, st, pred, gt, best, max_accept, cache_length,
                       kv_len, next_position_ids, result, flags);
    CPMCU_LAUNCH_CHECK();
    return CPMCU_OK;
}

extern "C" int cpmcu_verify_tail(void* const* k_pools, void* const* v_pools, int num_layers, const int32_t* block_table, int Hkv,
                                 int T, const int32_t* draft_ids, const int32_t* gt, const void* head_partials, int num_partials,
                                 int partial_stride, const int32_t* position_ids, const int32_t* cache_length,
                                 const uint64_t* attn_mask, int mask_words, const int32_t* tree_parent, const void* hidden,
                                 int hidden_dim, void* prev_hidden, int32_t* gt_out, int32_t* best, int32_t* path,
                                 int32_t* accepted_ids, int32_t* next_position_ids, int32_t* result, void* stream) {
    CPMCU_CHECK_ARG(k_pools && v_pools && block_table && draft_ids && position_ids && cache_length && attn_mask && tree_parent,
                    "verify_tail: null pointer argument");
    CPMCU_CHECK_ARG(num_layers >= 1 && Hkv >= 1, "verify_tail: num_layers=%d Hkv=%d", num_layers, Hkv);
    CPMCU_CHECK_ARG(T >= 1 && T <= kMaxTree, "verify_tail: tree size %d outside [1, %d]", T, kMaxTree);
    CPMCU_CHECK_ARG(mask_words >= 1 && mask_words <= 2 && mask_words * 64 >= T, "verify_tail: mask_words=%d does not cover T=%d", mask_words, T);
    CPMCU_CHECK_ARG((gt != nullptr) != (head_partials != nullptr), "verify_tail: give either gt or the head's partials");
    if (head_partials) {
        const bool pow2 = partial_stride >= 16 && partial_stride <= 128 && (partial_stride & (partial_stride - 1)) == 0;
        CPMCU_CHECK_ARG(pow2 && partial_stride >= T && num_partials >= 1 && num_partials <= head_max_grid(),
                        "verify_tail: %d partials of stride %d do not describe a head launch on %d rows", num_partials, partial_stride, T);
    }
    CPMCU_CHECK_ARG((hidden == nullptr) == (prev_hidden == nullptr), "verify_tail: hidden and prev_hidden go together");
    CPMCU_CHECK_ARG(hidden == nullptr || hidden != prev_hidden, "verify_tail: prev_hidden must not alias hidden");
    CPMCU_CHECK_ARG(!hidden || (hidden_dim >= 8 && hidden_dim % 8 == 0), "verify_tail: hidden_dim=%d must be a positive multiple of 8", hidden_dim);
    TailParams p;
    p.T = T;
    p.W = mask_words;
    p.draft = draft_ids;
    p.gt = gt;
    p.part_a = (const float*)head_partials;
    p.part_b = head_partials ? (const float*)head_partials + (size_t)head_max_grid() * 128 : nullptr;
    p.num_partials = num_partials;
    p.partial_stride = partial_stride;
    p.pos = position_ids;
    p.cache_length = cache_length;
    p.mask = attn_mask;
    p.parent = tree_parent;
    p.k_pools = k_pools;
    p.v_pools = v_pools;
    p.block_table = block_table;
    p.Hkv = Hkv;
    p.num_cache_blocks = num_layers * 2 * Hkv;
    p.hidden = (const f16x8*)hidden;
    p.prev_hidden = (f16x8*)prev_hidden;
    p.hidden_pieces = hidden ? hidden_dim / 8 : 0;
    p.num_hidden_blocks = hidden ? T : 0;
    p.gt_out = gt_out;
    p.best = best;
    p.path = path;
    p.ids = accepted_ids;
    p.next_position_ids = next_position_ids;
    p.result = result;
    hipLaunchKernelGGL(verify_tail_kernel, dim3(p.num_cache_blocks + p.num_hidden_blocks + 1), dim3(kTailThreads), 0, resolve_stream(stream), p);
    CPMCU_LAUNCH_CHECK();
    return CPMCU_OK;
}

extern "C" int cpmcu_verify_tail_inplace(const int32_t* best, const int32_t* accepted_ids, int T, int32_t* pred, int32_t* cache_length,
                                         int32_t* kv_len, int32_t* position_ids, int flags, void* stream) {
    CPMCU_CHECK_ARG(best && accepted_ids, "verify_tail_inplace: null pointer argument");
    CPMCU_CHECK_ARG(T >= 1 && T <= kMaxTree, "verify_tail_inplace: tree size %d outside [1, %d]", T, kMaxTree);
    CPMCU_CHECK_ARG((flags & ~(CPMCU_COMMIT_ADVANCE_LENGTH | CPMCU_COMMIT_NEXT_ROOT)) == 0, "verify_tail_inplace: unknown flags 0x%x", flags);
    CPMCU_CHECK_ARG(!(flags & CPMCU_COMMIT_ADVANCE_LENGTH) || cache_length, "verify_tail_inplace: the length advance needs cache_length");
    CPMCU_CHECK_ARG(!(flags & CPMCU_COMMIT_NEXT_ROOT) || pred, "verify_tail_inplace: the next root goes into pred");
    hipLaunchKernelGGL(verify_tail_inplace_kernel, dim3(1), dim3(128), 0, resolve_stream(stream), best, accepted_ids, T, pred, cache_length,
                       kv_len, position_ids, flags);
    CPMCU_LAUNCH_CHECK();
    return CPMCU_OK;
}

extern "C" int cpmcu_kv_append(void* k_pool, void* v_pool, const int32_t* block_table, const void* k_new,
                               const void* v_new, const int32_t* kv_len, int T, int Hkv, void* stream) {
    CPMCU_CHECK_ARG(k_pool && v_pool && block_table && k_new && v_new && kv_len, "kv_append: null pointer argument");
    CPMCU_CHECK_ARG(T >= 1 && Hkv >= 1, "kv_append: T=%d Hkv=%d", T, Hkv);
    hipLaunchKernelGGL(kv_append_kernel, dim3(T), dim3(256), 0, resolve_stream(stream), (f16*)k_pool, (f16*)v_pool,
                       block_table, (const f16*)k_new, (const f16*)v_new, kv_len, T, Hkv);
    CPMCU_LAUNCH_CHECK();
    return CPMCU_OK;
}
