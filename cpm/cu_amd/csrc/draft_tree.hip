// Draft-tree construction around the FR-Spec head for gfx950: the tree bookkeeping of the
// reference's draft() (src/model/minicpm4/minicpm4_eagle.cuh:319-393) as three single-workgroup
// kernels that keep all state on the device:
//   begin  -- d = 0: record the first k candidates, init_tree (src/model/eagle.cuh:91-93);
//   extend -- d >= 1: cumsum (eagle.cuh:103-106), history append, top-k over k*k -> k,
//             set_parent / update_tree (eagle.cuh:95-101), id remap (eagle.cuh:121-127) and the row
//             indices the hidden-state gather needs (remap_hidden, eagle.cuh:108-115);
//   finish -- top-(T-1) over the whole history, build_dynamic_tree (eagle.cuh:188-214) and the id
//             remap of the chosen nodes.
// The reference spends about ten launches and a device-to-host copy per iteration on these; here
// the prefix length is read from device memory, so building the tree needs no host round trip.
// Selection follows the ordering of the top-k kernels (value descending, lower index first).  The
// histories are short (k*k = 100 and k + 5*k*k = 510 entries at the reference's settings), so it is
// done by counting: every entry becomes a unique 32-bit key in LDS, every thread counts the keys above
// its own, and that count is the entry's place in the sorted order -- no rounds, two barriers.
#include "common.h"
#include "internal.h"
#include "topk_keys.h"

namespace cpmcu {
namespace {

constexpr int kMaxK = 32;        // topk_per_iter
constexpr int kMaxTried = kTopkThreads * kPerThread;  // history entries one workgroup can rank

// (order-preserving 16-bit image of the fp16 value) << 16 | (0xFFFF - index): unique, never 0 for index < kMaxTried.
__device__ inline uint32_t key32(uint16_t bits, int idx) { return (ord16(bits) << 16) | (uint32_t)(0xFFFF - idx); }
static_assert(kMaxTried <= 0x10000, "the index must fit the low half of a 32-bit key");

// Places of the `top` largest of s_keys[0, n): emit(place, index) is called by the thread that owns the
// entry.  s_keys must be padded with zeros to a multiple of 4 and be visible (barrier) on entry.
template <typename Emit>
__device__ inline void rank_select(const uint32_t* s_keys, int n, int top, Emit emit) {
    const int n4 = (n + 3) & ~3;
    for (int x = threadIdx.x; x < n; x += blockDim.x) {
        const uint32_t mine = s_keys[x];
        int above = 0;
#pragma unroll 8
        for (int j = 0; j < n4; j += 4) {  // every lane reads the same 16 bytes: an LDS broadcast
            const uint4 o = *reinterpret_cast<const uint4*>(s_keys + j);
            above += (o.x > mine) + (o.y > mine) + (o.z > mine) + (o.w > mine);
        }
        if (above < top) emit(above, x);
    }
}

struct DraftState {
    uint16_t* tried_val;    // [total] fp16 bits
    int32_t* tried_pos;     // [total]
    int32_t* tried_parent;  // [k * (num_iter - 1)]
    uint64_t* mask;         // [k] eagle_mask_2d
    uint16_t* cum;          // [k] running log-prob of the k live nodes
};

__host__ __device__ inline size_t draft_state_layout(int k, int num_iter, size_t* off_pos, size_t* off_parent, size_t* off_mask,
                                                     size_t* off_cum) {
    const size_t total = (size_t)k + (size_t)(num_iter - 1) * k * k;
    size_t o = (total * 2 + 15) / 16 * 16;
    *off_pos = o;
    o += total * 4;
    *off_parent = o;
    o += (size_t)k * (num_iter > 1 ? num_iter - 1 : 1) * 4;
    o = (o + 15) / 16 * 16;
    *off_mask = o;
    o += (size_t)k * 8;
    *off_cum = o;
    o += (size_t)k * 2;
    return (o + 255) / 256 * 256;
}

inline DraftState draft_state(void* state, int k, int num_iter) {
    size_t op, opar, om, oc;
    draft_state_layout(k, num_iter, &op, &opar, &om, &oc);
    char* b = (char*)state;
    return DraftState{(uint16_t*)b, (int32_t*)(b + op), (int32_t*)(b + opar), (uint64_t*)(b + om), (uint16_t*)(b + oc)};
}

__global__ void draft_begin_kernel(DraftState s, int k, const uint16_t* val, const int32_t* pos, const int32_t* remap,
                                   int32_t* next_ids, uint64_t* mask_out) {
    const int i = threadIdx.x;
    if (i >= k) return;
    s.tried_val[i] = val[i];
    s.tried_pos[i] = pos[i];
    s.cum[i] = val[i];
    s.mask[i] = 1ull << i;
    if (mask_out) mask_out[i] = 1ull << i;
    next_ids[i] = remap ? remap[pos[i]] : pos[i];
}

__global__ __launch_bounds__(kTopkThreads) void draft_extend_kernel(DraftState s, int k, int d, uint16_t* val, const int32_t* pos,
                                                                    const int32_t* remap, int32_t* next_ids, int32_t* parent_rows,
                                                                    uint64_t* mask_out, int is_bf16) {
    __shared__ __attribute__((aligned(16))) uint32_t s_keys[kMaxK * kMaxK];
    __shared__ int32_t s_sel[kMaxK];
    __shared__ uint16_t s_val[kMaxK * kMaxK];
    __shared__ uint64_t s_oldmask[kMaxK];
    const int tid = threadIdx.x;
    const int kk = k * k;
    const int base = k + (d - 1) * kk;
    if (tid < k) s_oldmask[tid] = s.mask[tid];
    for (int x = tid; x < ((kk + 3) & ~3); x += kTopkThreads) {
        uint32_t key = 0;
        if (x < kk) {
            // the running log-prob of the parent is added in the element type: 16 bits += 16 bits, rounded to 16 bits
            const uint16_t bits = is_bf16 ? Elem<bf16>::to_bits(Elem<bf16>::from_bits(val[x]) + Elem<bf16>::from_bits(s.cum[x / k]))
                                          : Elem<f16>::to_bits(Elem<f16>::from_bits(val[x]) + Elem<f16>::from_bits(s.cum[x / k]));
            val[x] = bits;
            s.tried_val[base + x] = bits;
            s.tried_pos[base + x] = pos[x];
            s_val[x] = bits;
            key = key32(bits, x);
        }
        s_keys[x] = key;
    }
    __syncthreads();
    rank_select(s_keys, kk, k, [&](int place, int x) { s_sel[place] = x; });
    __syncthreads();
    if (tid < k) {
        const int p2 = s_sel[tid];
        s.tried_parent[(d - 1) * k + tid] = p2 + base;
        const uint64_t m = s_oldmask[p2 / k] | (1ull << (k * d + tid));
        s.mask[tid] = m;
        if (mask_out) mask_out[tid] = m;
        if (parent_rows) parent_rows[tid] = p2 / k;
        const int32_t fr = pos[p2];
        next_ids[tid] = remap ? remap[fr] : fr;
        s.cum[tid] = s_val[p2];
    }
}

// One thread per history entry up to 1024 entries (two beyond): the counting loop is a chain of LDS
// reads, and sixteen waves hide its latency where four would wait for it.
constexpr int kFinishThreads = 1024;

__global__ __launch_bounds__(kFinishThreads) void draft_finish_kernel(DraftState s, int k, int num_iter, int T, const int32_t* cache_length,
                                                                      const int32_t* remap, int32_t* ids_out, int32_t* tree_pos,
                                                                      uint64_t* tree_mask, int32_t* tree_parent) {
    __shared__ __attribute__((aligned(16))) uint32_t s_keys[kMaxTried];
    __shared__ int32_t s_pos[kMaxTried];     // FR-Spec index of every history entry
    __shared__ int32_t s_reverse[kMaxTried]; // history index -> tree node (0: not selected, stands for the root)
    __shared__ int32_t s_hpar[64];           // history parent of the entries chosen in rounds >= 1 (k * num_iter <= 64 of them)
    __shared__ int32_t s_sel[kMaxTree];      // history index of tree node i + 1
    __shared__ int32_t s_par[kMaxTree];
    const int tid = threadIdx.x;
    const int kk = k * k;
    const int total = k + (num_iter - 1) * kk;
    const int W = (T + 63) / 64;
    // everything the later phases need comes into LDS in one round trip to memory
    for (int x = tid; x < ((total + 3) & ~3); x += kFinishThreads) {
        const bool in = x < total;
        s_keys[x] = in ? key32(s.tried_val[x], x) : 0;
        if (in) {
            s_pos[x] = s.tried_pos[x];
            s_reverse[x] = 0;  // a parent that was not selected maps to the root
        }
    }
    if (tid < k * (num_iter - 1)) s_hpar[tid] = s.tried_parent[tid];
    const int P = cache_length[0];
    __syncthreads();
    rank_select(s_keys, total, T - 1, [&](int place, int x) { s_sel[place] = x; });
    __syncthreads();
    if (tid >= 1 && tid < T) {
        const int p = s_sel[tid - 1];
        s_reverse[p] = tid;
        const int32_t fr = s_pos[p];
        ids_out[tid] = remap ? remap[fr] : fr;
    }
    __syncthreads();
    // build_dynamic_tree (src/model/eagle.cuh:188-214), every node on its own thread: its parent is the
    // tree node of its history parent; its mask row is its own bit plus those of its ancestors.
    // Parents come before children (cumulative log-probs fall along a path, ties go to the older
    // entry), which the sequential form of the reference relies on as well.
    if (tid < T) {
        int parent = 0;
        if (tid == 0) {
            tree_pos[0] = P;
        } else {
            int p = s_sel[tid - 1];
            tree_pos[tid] = P + (p < k ? 1 : (p - k) / kk + 2);
            if (p >= k) {
                p -= k;
                p = p < kk ? p / k : s_hpar[(p - kk) / k];
                parent = s_reverse[p];
            }
        }
        s_par[tid] = parent;
        tree_parent[tid] = parent;
    }
    __syncthreads();
    if (tid < T) {
        uint64_t m0 = 1, m1 = 0;  // the root is everybody's ancestor
        int node = tid;
        for (int hop = 0; hop < T && node != 0; ++hop) {
            if (node < 64) m0 |= 1ull << node;
            else m1 |= 1ull << (node - 64);
            const int up = s_par[node];
            node = up < node ? up : 0;  // never walks downwards, so it ends
        }
        tree_mask[(size_t)tid * W] = m0;
        if (W > 1) tree_mask[(size_t)tid * W + 1] = m1;
    }
}

int check_shape(const char* what, int k, int num_iter) {
    CPMCU_CHECK_ARG(k >= 1 && k <= kMaxK, "%s: k=%d outside [1, %d]", what, k, kMaxK);
    CPMCU_CHECK_ARG(num_iter >= 1 && k * num_iter <= 64, "%s: k * num_iter = %d does not fit the 64-bit draft mask", what, k * num_iter);
    CPMCU_CHECK_ARG((size_t)k + (size_t)(num_iter - 1) * k * k <= (size_t)kMaxTried, "%s: history of %d entries exceeds %d", what,
                    k + (num_iter - 1) * k * k, kMaxTried);
    return CPMCU_OK;
}

}  // namespace
}  // namespace cpmcu

using namespace cpmcu;

extern "C" size_t cpmcu_draft_tree_state_bytes(int k, int num_iter) {
    if (k < 1 || num_iter < 1) return 0;
    size_t a, b, c, d;
    return draft_state_layout(k, num_iter, &a, &b, &c, &d);
}

extern "C" int cpmcu_draft_tree_begin(void* state, int k, int num_iter, const void* topk_val, const int32_t* topk_pos,
                                      const int32_t* token_id_remap, int32_t* next_ids, uint64_t* draft_mask, void* stream) {
    CPMCU_CHECK_ARG(state && topk_val && topk_pos && next_ids, "draft_tree_begin: null pointer argument");
    if (int rc = check_shape("draft_tree_begin", k, num_iter)) return rc;
    hipLaunchKernelGGL(draft_begin_kernel, dim3(1), dim3(64), 0, resolve_stream(stream), draft_state(state, k, num_iter), k,
                       (const uint16_t*)topk_val, topk_pos, token_id_remap, next_ids, draft_mask);
    CPMCU_LAUNCH_CHECK();
    return CPMCU_OK;
}

extern "C" int cpmcu_draft_tree_extend(void* state, int k, int num_iter, int d, void* topk_val, const int32_t* topk_pos,
                                       const int32_t* token_id_remap, int32_t* next_ids, int32_t* parent_rows,
                                       uint64_t* draft_mask, void* stream) {
    CPMCU_CHECK_ARG(state && topk_val && topk_pos && next_ids, "draft_tree_extend: null pointer argument");
    if (int rc = check_shape("draft_tree_extend", k, num_iter)) return rc;
    CPMCU_CHECK_ARG(d >= 1 && d < num_iter, "draft_tree_extend: iteration d=%d outside [1, %d)", d, num_iter);
    hipLaunchKernelGGL(draft_extend_kernel, dim3(1), dim3(kTopkThreads), 0, resolve_stream(stream), draft_state(state, k, num_iter), k, d,
                       (uint16_t*)topk_val, topk_pos, token_id_remap, next_ids, parent_rows, draft_mask, options().dtype == 1 ? 1 : 0);
    CPMCU_LAUNCH_CHECK();
    return CPMCU_OK;
}

extern "C" int cpmcu_draft_tree_finish(void* state, int k, int num_iter, int tree_size, const int32_t* cache_length,
                                       const int32_t* token_id_remap, int32_t* tree_draft_ids, int32_t* tree_position_ids,
                                       uint64_t* tree_attn_mask, int32_t* tree_parent, void* stream) {
    CPMCU_CHECK_ARG(state && cache_length && tree_draft_ids && tree_position_ids && tree_attn_mask && tree_parent,
                    "draft_tree_finish: null pointer argument");
    if (int rc = check_shape("draft_tree_finish", k, num_iter)) return rc;
    const int total = k + (num_iter - 1) * k * k;
    CPMCU_CHECK_ARG(tree_size >= 2 && tree_size <= kMaxTree && tree_size - 1 <= total,
                    "draft_tree_finish: tree_size=%d outside [2, min(%d, history %d + 1)]", tree_size, kMaxTree, total);
    hipLaunchKernelGGL(draft_finish_kernel, dim3(1), dim3(kFinishThreads), 0, resolve_stream(stream), draft_state(state, k, num_iter), k,
                       num_iter, tree_size, cache_length, token_id_remap, tree_draft_ids, tree_position_ids, tree_attn_mask, tree_parent);
    CPMCU_LAUNCH_CHECK();
    return CPMCU_OK;
}
