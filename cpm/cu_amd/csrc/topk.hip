// Exact top-k, log-softmax, FR-Spec id map-back and row gather for gfx950.
//
// Ordering contract of the reference's bitonic TopK (src/model/topk.cuh:17): value descending,
// equal values -> lower index first.  Here every element becomes one 64-bit key
//   (order-preserving 16-bit image of the fp16 value) << 32 | (0xFFFFFFFF - index)
// so "largest key first" IS that ordering, keys are unique, and selection is k rounds of a
// workgroup-wide max -- no sorting network, no padding to powers of two, any k.
//
// FR-Spec fusion: the draft head ranks log-probabilities that were rounded to fp16 BEFORE
// ranking (src/model/eagle.cuh:87), so rounding ties must be reproduced exactly.  The chunk
// kernel therefore recomputes f16((z - max) - ln sum) from the fp16 logits and the row
// statistics reduced from the GEMM's per-workgroup partials, and ranks that.
#include "common.h"
#include "internal.h"
#include "topk_keys.h"

namespace cpmcu {
namespace {

struct TopkParams {
    const uint16_t* x;  // [n][dim] fp16 bits
    int n, dim, top, nchunks;
    uint64_t* cand;     // [n][nchunks][top]
    uint16_t* val;      // [n][top]
    int32_t* pos;
    int32_t* ids;
    const int32_t* remap;
    // fused log-softmax
    const float* part_max;
    const float* part_sum;
    int grid, stride;
    float* row_stats;
};

template <bool LOGSOFTMAX>
__device__ inline void emit_final(const TopkParams& p, int row, int round, uint64_t key) {
    if (key == 0) return;
    const int idx = key_index(key);
    const size_t o = (size_t)row * p.top + round;
    // raw ranking: hand back the input bits (keeps -0); fused: the rounded log-prob in the key
    p.val[o] = LOGSOFTMAX ? key_bits(key) : p.x[(size_t)row * p.dim + idx];
    p.pos[o] = idx;
    if (p.ids) p.ids[o] = p.remap ? p.remap[idx] : idx;
}

template <bool LOGSOFTMAX>
__global__ __launch_bounds__(kTopkThreads) void topk_chunk_kernel(TopkParams p) {
    const int chunk = blockIdx.x;
    const int row = blockIdx.y;
    const int tid = threadIdx.x;
    float m = 0.f, lse = 0.f;
    if (LOGSOFTMAX) {
        // row statistics from the GEMM's per-workgroup (max, sum exp(z - max)) partials: in-wave by
        // shuffles, then across the four waves through LDS
        __shared__ float sm[kTopkThreads / 64], ss[kTopkThreads / 64];
        float a = -INFINITY, b = 0.f;
        for (int c = tid; c < p.grid; c += kTopkThreads) {
            const float oa = p.part_max[(size_t)c * p.stride + row];
            const float ob = p.part_sum[(size_t)c * p.stride + row];
            const float mm = fmaxf(a, oa);
            b = (mm == -INFINITY) ? 0.f : b * expf(a - mm) + ob * expf(oa - mm);
            a = mm;
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
            const float oa = __shfl_xor(a, off), ob = __shfl_xor(b, off);
            const float mm = fmaxf(a, oa);
            b = (mm == -INFINITY) ? 0.f : b * expf(a - mm) + ob * expf(oa - mm);
            a = mm;
        }
        if ((tid & 63) == 0) {
            sm[tid >> 6] = a;
            ss[tid >> 6] = b;
        }
        __syncthreads();
        a = sm[0];
        b = ss[0];
#pragma unroll
        for (int w = 1; w < kTopkThreads / 64; ++w) {
            const float mm = fmaxf(a, sm[w]);
            b = (mm == -INFINITY) ? 0.f : b * expf(a - mm) + ss[w] * expf(sm[w] - mm);
            a = mm;
        }
        m = a;
        lse = logf(b);
        if (chunk == 0 && tid == 0 && p.row_stats) {
            p.row_stats[row * 2 + 0] = m;
            p.row_stats[row * 2 + 1] = lse;
        }
    }
    uint64_t keys[kPerThread];
    const int base = chunk * kChunk + tid * kPerThread;
    const uint16_t* xr = p.x + (size_t)row * p.dim;
#pragma unroll
    for (int e = 0; e < kPerThread; ++e) {
        const int idx = base + e;
        uint64_t key = 0;
        if (idx < p.dim) {
            uint16_t bits = xr[idx];
            if (LOGSOFTMAX) {
                const float z = (float)__builtin_bit_cast(f16, bits);
                const f16 lp = (f16)((z - m) - lse);  // src/model/eagle.cuh:87
                bits = __builtin_bit_cast(uint16_t, lp);
            }
            key = make_key(bits, idx);
        }
        keys[e] = key;
    }
    if (p.nchunks == 1) {
        select_topk(keys, p.top, [&](int round, uint64_t key) { emit_final<LOGSOFTMAX>(p, row, round, key); });
    } else {
        uint64_t* out = p.cand + ((size_t)row * p.nchunks + chunk) * p.top;
        select_topk(keys, p.top, [&](int round, uint64_t key) { out[round] = key; });
    }
}

template <bool LOGSOFTMAX>
__global__ __launch_bounds__(kTopkThreads) void topk_merge_kernel(TopkParams p) {
    const int row = blockIdx.x;
    const int ncand = p.nchunks * p.top;
    const uint64_t* in = p.cand + (size_t)row * ncand;
    uint64_t keys[kPerThread];
#pragma unroll
    for (int e = 0; e < kPerThread; ++e) {
        const int i = threadIdx.x + e * kTopkThreads;
        keys[e] = i < ncand ? in[i] : 0;
    }
    select_topk(keys, p.top, [&](int round, uint64_t key) { emit_final<LOGSOFTMAX>(p, row, round, key); });
}

// log_softmax in place (src/model/eagle.cuh:29-89): one workgroup per row.
__global__ __launch_bounds__(1024) void log_softmax_kernel(uint16_t* x, int dim, float* row_stats) {
    __shared__ float red[16];
    const int row = blockIdx.x;
    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    uint16_t* xr = x + (size_t)row * dim;
    float m = -INFINITY;
    for (int i = tid; i < dim; i += 1024) m = fmaxf(m, (float)__builtin_bit_cast(f16, xr[i]));
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) m = fmaxf(m, __shfl_xor(m, off));
    if (lane == 0) red[wave] = m;
    __syncthreads();
    m = red[0];
#pragma unroll
    for (int w = 1; w < 16; ++w) m = fmaxf(m, red[w]);
    __syncthreads();
    float s = 0.f;
    for (int i = tid; i < dim; i += 1024) s += expf((float)__builtin_bit_cast(f16, xr[i]) - m);
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) s += __shfl_xor(s, off);
    if (lane == 0) red[wave] = s;
    __syncthreads();
    s = 0.f;
#pragma unroll
    for (int w = 0; w < 16; ++w) s += red[w];
    const float lse = logf(s);
    for (int i = tid; i < dim; i += 1024) {
        const f16 lp = (f16)(((float)__builtin_bit_cast(f16, xr[i]) - m) - lse);
        xr[i] = __builtin_bit_cast(uint16_t, lp);
    }
    if (tid == 0 && row_stats) {
        row_stats[row * 2 + 0] = m;
        row_stats[row * 2 + 1] = lse;
    }
}

__global__ void remap_kernel(const int32_t* in, int n, const int32_t* table, int32_t* out) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = table[in[i]];
}

// remap_copy (src/model/tree_drafter.cuh:79-86): one workgroup per destination row, 16-byte pieces.
__global__ __launch_bounds__(256) void gather_rows_kernel(const f16x8* src, const int32_t* remap, int dim8, f16x8* dst) {
    const int row = blockIdx.x;
    const size_t s = (size_t)remap[row] * dim8;
    const size_t d = (size_t)row * dim8;
    for (int i = threadIdx.x; i < dim8; i += 256) dst[d + i] = src[s + i];
}

}  // namespace

int launch_topk(const void* x, int n, int dim, int top, void* val, int32_t* pos, int32_t* ids,
                const int32_t* token_id_remap, const TopkStatsSource* stats, void* workspace,
                size_t workspace_bytes, hipStream_t st) {
    TopkParams p;
    p.x = (const uint16_t*)x;
    p.n = n;
    p.dim = dim;
    p.top = top;
    p.nchunks = ceil_div(dim, kChunk);
    CPMCU_CHECK_ARG(p.nchunks * top <= kMaxCand, "topk: dim=%d with top=%d needs %d merge candidates, limit %d",
                    dim, top, p.nchunks * top, kMaxCand);
    p.cand = (uint64_t*)workspace;
    p.val = (uint16_t*)val;
    p.pos = pos;
    p.ids = ids;
    p.remap = token_id_remap;
    p.part_max = stats ? stats->part_max : nullptr;
    p.part_sum = stats ? stats->part_sum : nullptr;
    p.grid = stats ? stats->grid : 0;
    p.stride = stats ? stats->stride : 0;
    p.row_stats = stats ? stats->row_stats : nullptr;
    if (p.nchunks > 1) {
        const size_t need = (size_t)n * p.nchunks * top * sizeof(uint64_t);
        CPMCU_CHECK_ARG(workspace && workspace_bytes >= need, "topk: workspace of %zu bytes needed, %zu given", need, workspace_bytes);
    }
    const dim3 grid(p.nchunks, n);
    if (stats) {
        hipLaunchKernelGGL(topk_chunk_kernel<true>, grid, dim3(kTopkThreads), 0, st, p);
        CPMCU_LAUNCH_CHECK();
        if (p.nchunks > 1) {
            hipLaunchKernelGGL(topk_merge_kernel<true>, dim3(n), dim3(kTopkThreads), 0, st, p);
            CPMCU_LAUNCH_CHECK();
        }
    } else {
        hipLaunchKernelGGL(topk_chunk_kernel<false>, grid, dim3(kTopkThreads), 0, st, p);
        CPMCU_LAUNCH_CHECK();
        if (p.nchunks > 1) {
            hipLaunchKernelGGL(topk_merge_kernel<false>, dim3(n), dim3(kTopkThreads), 0, st, p);
            CPMCU_LAUNCH_CHECK();
        }
    }
    return CPMCU_OK;
}

}  // namespace cpmcu

using namespace cpmcu;

extern "C" size_t cpmcu_topk_workspace_bytes(int n, int dim, int top) {
    if (n <= 0 || dim <= 0 || top <= 0) return 0;
    return align_up((size_t)n * ceil_div(dim, kChunk) * top * sizeof(uint64_t), 256);
}

extern "C" int cpmcu_topk(const void* x, int n, int dim, int top, void* val, int32_t* pos, void* workspace,
                          size_t workspace_bytes, void* stream) {
    CPMCU_CHECK_ARG(x && val && pos, "topk: null pointer argument");
    CPMCU_CHECK_ARG(n >= 1 && dim >= 1, "topk: bad shape n=%d dim=%d", n, dim);
    CPMCU_CHECK_ARG(top >= 1 && top <= dim && top <= 128, "topk: top=%d outside [1, min(dim=%d, 128)]", top, dim);
    return launch_topk(x, n, dim, top, val, pos, nullptr, nullptr, nullptr, workspace, workspace_bytes, resolve_stream(stream));
}

extern "C" int cpmcu_log_softmax(void* x, int n, int dim, float* row_stats, void* stream) {
    CPMCU_CHECK_ARG(x, "log_softmax: null pointer argument");
    CPMCU_CHECK_ARG(n >= 1 && dim >= 1, "log_softmax: bad shape n=%d dim=%d", n, dim);
    hipLaunchKernelGGL(log_softmax_kernel, dim3(n), dim3(1024), 0, resolve_stream(stream), (uint16_t*)x, dim, row_stats);
    CPMCU_LAUNCH_CHECK();
    return CPMCU_OK;
}

extern "C" int cpmcu_remap(const int32_t* in, int n, const int32_t* token_id_remap, int32_t* out, void* stream) {
    CPMCU_CHECK_ARG(in && token_id_remap && out, "remap: null pointer argument");
    CPMCU_CHECK_ARG(n >= 1, "remap: n=%d", n);
    hipLaunchKernelGGL(remap_kernel, dim3(ceil_div(n, 256)), dim3(256), 0, resolve_stream(stream), in, n, token_id_remap, out);
    CPMCU_LAUNCH_CHECK();
    return CPMCU_OK;
}

extern "C" int cpmcu_gather_rows(const void* src, const int32_t* remap, int rows, int dim, void* dst, void* stream) {
    CPMCU_CHECK_ARG(src && remap && dst, "gather_rows: null pointer argument");
    CPMCU_CHECK_ARG(rows >= 1 && dim >= 8 && dim % 8 == 0, "gather_rows: rows=%d, dim=%d must be a positive multiple of 8", rows, dim);
    hipLaunchKernelGGL(gather_rows_kernel, dim3(rows), dim3(256), 0, resolve_stream(stream), (const f16x8*)src, remap, dim / 8, (f16x8*)dst);
    CPMCU_LAUNCH_CHECK();
    return CPMCU_OK;
}

extern "C" int cpmcu_frspec_head_topk(const void* hidden, const void* w, int w_layout, const int32_t* token_id_remap, int n, int V,
                                      int H, int k, void* logits, float* row_stats, void* topk_val,
                                      int32_t* topk_pos, int32_t* topk_ids, void* workspace, size_t workspace_bytes,
                                      void* stream) {
    CPMCU_CHECK_ARG(hidden && w && logits && topk_val && topk_pos, "frspec_head_topk: null pointer argument");
    CPMCU_CHECK_ARG(n >= 1 && n <= 16, "frspec_head_topk: n=%d outside [1, 16]", n);
    CPMCU_CHECK_ARG(k >= 1 && k <= 32 && k <= V, "frspec_head_topk: k=%d outside [1, min(32, V=%d)]", k, V);
    CPMCU_CHECK_ARG(workspace && workspace_bytes >= cpmcu_head_workspace_bytes(n, V),
                    "frspec_head_topk: workspace of %zu bytes needed, %zu given", cpmcu_head_workspace_bytes(n, V), workspace_bytes);
    hipStream_t st = resolve_stream(stream);
    float* part_a = (float*)workspace;
    float* part_b = part_a + (size_t)head_max_grid() * 128;
    const size_t parts_bytes = align_up((size_t)2 * head_max_grid() * 128 * sizeof(float), 256);
    int G = 0, stride = 0;
    int rc = launch_head_gemm(hidden, w, w_layout, n, V, H, 0, 1.f, kHeadModeStats, logits, part_a, part_b, &G, &stride, st);
    if (rc != CPMCU_OK) return rc;
    TopkStatsSource src{part_a, part_b, G, stride, row_stats};
    return launch_topk(logits, n, V, k, topk_val, topk_pos, topk_ids, token_id_remap, &src,
                       (char*)workspace + parts_bytes, workspace_bytes - parts_bytes, st);
}
