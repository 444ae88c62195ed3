// Tree-verify flash attention for gfx950 (MI355X): tree-masked draft queries
// against the paged prefix KV plus the in-tree KV, GQA-packed, fp16 MFMA with
// fp32 accumulation, split over the KV stream and merged by a second kernel.
//
// What it computes is the dense tree-mask path of the reference's
// mha_fwd_kvcache (src/flash_attn/flash_api.hpp:292-392, kernel body
// src/flash_attn/src/flash_fwd_kernel.h:1175-1766, mask src/flash_attn/src/mask.h:139-229,
// merge src/flash_attn/src/flash_fwd_kernel.h:2320-2501).  How it computes it is
// specific to CDNA4:
//
//  * GQA packing: the `group` query heads that share a KV head and the T tree
//    nodes form one M = group*T row matrix per KV head (node-major), so every
//    K/V tile fetched from HBM feeds group*T query rows instead of T.
//  * The scores are produced transposed, S^T = K.Q^T, with
//    v_mfma_f32_32x32x16_f16: each lane then owns ONE query column and 16 key
//    rows per 32x32 block, so the online-softmax row reductions are in-lane
//    plus a single cross-half exchange, and the fp16 probabilities are already
//    in the B-operand layout of the second product O^T = V^T.P^T -- no LDS
//    round trip for P.
//  * V pages are stored transposed and 16-token interleaved (see
//    include/cpmcu_amd.h) so the A operand of O^T = V^T.P^T is one 16-byte LDS
//    read per lane.
//  * Workgroups are mapped so that all M-tiles that stream the same KV range
//    land on the same XCD (workgroup id modulo 8) and share its L2.
#include "common.h"

namespace cpmcu {
namespace {

constexpr int kTileN = 64;                     // keys per LDS tile
constexpr int kWaves = 4;                      // waves per workgroup
constexpr int kRowsPerWave = 32;               // packed query rows per wave (one MFMA N block)
constexpr int kRowsPerWg = kWaves * kRowsPerWave;
constexpr int kThreads = kWaves * 64;
constexpr int kKRowBytes = kHeadDim * 2 + 16;  // padded K row in LDS: conflict-free b128 reads
constexpr int kVRowBytes = kTileN * 2 + 16;    // padded V^T row in LDS
constexpr int kXcds = 8;

struct AttnParams {
    const f16* q;
    const f16* k_pool;
    const f16* v_pool;
    const int32_t* block_table;
    const int32_t* kv_len;
    const uint64_t* mask;
    int mask_words;
    int T, Hq, Hkv, group;
    int num_splits, num_mtiles, rows_pad;
    float scale_log2;
    f16* out;
    float* o_part;   // [Hkv][num_splits][rows_pad][128]
    float* ml_part;  // [Hkv][num_splits][rows_pad][2]  (max * scale_log2, sum)
};

__device__ inline f16x8 zero8() {
    f16x8 z;
#pragma unroll
    for (int i = 0; i < 8; ++i) z[i] = (f16)0.f;
    return z;
}

struct TileRegs {
    f16x8 k[4];
    f16x8 v[4];
};

// Global -> registers for one 64-key tile.  Keys at or beyond S are zero-filled
// (stale or never-written page memory must not reach the MFMAs: 0 * NaN = NaN).
__device__ inline void load_tile(const AttnParams& p, int g, int tile, int S, int tid, TileRegs& r) {
    const int c0 = tile * kTileN;
    const int page = p.block_table[c0 / kPage];
    const int slot0 = c0 % kPage;
    const f16* kbase = p.k_pool + (((size_t)page * p.Hkv + g) * kPage + slot0) * kHeadDim;
    const f16* vbase = p.v_pool + ((size_t)page * p.Hkv + g) * kHeadDim * kPage + slot0;
    const bool partial = c0 + kTileN > S;
#pragma unroll
    for (int ps = 0; ps < 4; ++ps) {
        const int key = ps * 16 + (tid >> 4);
        const int chunk = tid & 15;
        if (!partial || c0 + key < S)
            r.k[ps] = *reinterpret_cast<const f16x8*>(kbase + (size_t)key * kHeadDim + chunk * 8);
        else
            r.k[ps] = zero8();
    }
#pragma unroll
    for (int ps = 0; ps < 4; ++ps) {
        const int d = ps * 32 + (tid >> 3);
        const int chunk = tid & 7;
        f16x8 v = *reinterpret_cast<const f16x8*>(vbase + (size_t)d * kPage + chunk * 8);
        if (partial) {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const int key = v_slot16(chunk * 8 + e);  // storage slot -> token within the tile
                if (c0 + key >= S) v[e] = (f16)0.f;
            }
        }
        r.v[ps] = v;
    }
}

__device__ inline void store_tile(char* lds_k, char* lds_v, int tid, const TileRegs& r) {
#pragma unroll
    for (int ps = 0; ps < 4; ++ps) {
        const int key = ps * 16 + (tid >> 4);
        const int chunk = tid & 15;
        *reinterpret_cast<f16x8*>(lds_k + key * kKRowBytes + chunk * 16) = r.k[ps];
    }
#pragma unroll
    for (int ps = 0; ps < 4; ++ps) {
        const int d = ps * 32 + (tid >> 3);
        const int chunk = tid & 7;
        *reinterpret_cast<f16x8*>(lds_v + d * kVRowBytes + chunk * 16) = r.v[ps];
    }
}

__global__ __launch_bounds__(kThreads) void tree_attn_split_kernel(AttnParams p) {
    __shared__ __attribute__((aligned(16))) char lds_k[kTileN * kKRowBytes];
    __shared__ __attribute__((aligned(16))) char lds_v[kHeadDim * kVRowBytes];

    // XCD-aware work mapping: consecutive workgroup ids go to consecutive XCDs, so
    // id % 8 picks the XCD; all M-tiles of one (split, kv head) pair share an XCD.
    const int wg = blockIdx.x;
    const int xcd = wg % kXcds;
    const int j = wg / kXcds;
    const int sh = xcd + kXcds * (j / p.num_mtiles);
    const int mt = j % p.num_mtiles;
    if (sh >= p.num_splits * p.Hkv) return;
    const int g = sh % p.Hkv;
    const int split = sh / p.Hkv;

    const int tid = threadIdx.x;
    const int wave = tid >> 6;
    const int lane = tid & 63;
    const int qcol = lane & 31;
    const int hf = lane >> 5;

    const int S = p.kv_len[0];
    const int P = S - p.T;
    const int ntiles = (S + kTileN - 1) / kTileN;
    const int tps = (ntiles + p.num_splits - 1) / p.num_splits;
    const int t0 = split * tps;
    const int t1 = min(ntiles, t0 + tps);

    const int R = mt * kRowsPerWg + wave * kRowsPerWave + qcol;  // packed row
    const bool row_ok = R < p.group * p.T;
    const int node = row_ok ? R / p.group : 0;
    const int head = g * p.group + (row_ok ? R % p.group : 0);

    // Q as the B operand of S^T = K.Q^T: lane (qcol, hf) holds d = 16*ks + 8*hf + [0,8).
    f16x8 qreg[8];
    {
        const f16* qrow = p.q + ((size_t)node * p.Hq + head) * kHeadDim + hf * 8;
#pragma unroll
        for (int ks = 0; ks < 8; ++ks)
            qreg[ks] = row_ok ? *reinterpret_cast<const f16x8*>(qrow + ks * 16) : zero8();
    }
    // Tree mask row of this lane's node with the causal bound j <= node folded in
    // (src/flash_attn/src/mask.h:185-198).
    uint64_t mw0, mw1 = 0;
    if (p.mask) {
        mw0 = p.mask[(size_t)node * p.mask_words];
        if (p.mask_words > 1) mw1 = p.mask[(size_t)node * p.mask_words + 1];
    } else {
        mw0 = ~0ull;
        mw1 = ~0ull;
    }
    {
        const uint64_t c0 = node >= 63 ? ~0ull : ((2ull << node) - 1ull);
        const uint64_t c1 = node >= 127 ? ~0ull : (node < 64 ? 0ull : ((2ull << (node - 64)) - 1ull));
        mw0 &= c0;
        mw1 &= c1;
    }

    f32x16 oacc[4];
#pragma unroll
    for (int db = 0; db < 4; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) oacc[db][r] = 0.f;
    float m_run = -INFINITY;  // running row max (raw score units)
    float l_run = 0.f;        // this lane's share of the row sum

    TileRegs regs;
    if (t0 < t1) load_tile(p, g, t0, S, tid, regs);

    for (int t = t0; t < t1; ++t) {
        __syncthreads();  // previous tile fully consumed
        store_tile(lds_k, lds_v, tid, regs);
        __syncthreads();
        if (t + 1 < t1) load_tile(p, g, t + 1, S, tid, regs);  // prefetch under the MFMAs

        // ---- S^T = K.Q^T : two 32-key blocks ----
        f32x16 sacc[2];
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
            for (int r = 0; r < 16; ++r) sacc[kb][r] = 0.f;
            const char* krow = lds_k + (kb * 32 + qcol) * kKRowBytes + hf * 16;
#pragma unroll
            for (int ks = 0; ks < 8; ++ks) {
                const f16x8 a = *reinterpret_cast<const f16x8*>(krow + ks * 32);
                sacc[kb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, qreg[ks], sacc[kb], 0, 0, 0);
            }
        }
        // sacc[kb][r] is the score of key  c0 + kb*32 + 8*(r/4) + 4*hf + r%4  for query qcol.
        const int c0 = t * kTileN;
        if (c0 + kTileN > P) {  // tile touches tree columns or the end of the stream
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int c = c0 + kb * 32 + 8 * (r >> 2) + 4 * hf + (r & 3);
                    const int jn = c - P;
                    bool vis = true;
                    if (jn >= 0) {
                        const uint64_t w = jn < 64 ? mw0 : mw1;
                        vis = jn < p.T && ((w >> (jn & 63)) & 1ull);
                    }
                    if (!vis) sacc[kb][r] = -INFINITY;
                }
        }
        // ---- online softmax (one query column per lane) ----
        float tmax = sacc[0][0];
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int r = 0; r < 16; ++r) tmax = fmaxf(tmax, sacc[kb][r]);
        tmax = fmaxf(tmax, __shfl_xor(tmax, 32));
        const float m_new = fmaxf(m_run, tmax);
        const float m_scaled = (m_new == -INFINITY) ? 0.f : m_new * p.scale_log2;
        const float alpha = __builtin_amdgcn_exp2f(m_run * p.scale_log2 - m_scaled);
        m_run = m_new;
        float psum = 0.f;
        f16x8 pb[4];  // P^T as B operand: k-step jj holds keys 16*jj + {4hf..4hf+3, 8+4hf..8+4hf+3}
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const float pv = __builtin_amdgcn_exp2f(sacc[kb][r] * p.scale_log2 - m_scaled);
                psum += pv;                                // row sum keeps the fp32 value
                pb[kb * 2 + (r >> 3)][r & 7] = (f16)pv;    // P is rounded to fp16 before P.V
            }
        l_run = l_run * alpha + psum;
#pragma unroll
        for (int db = 0; db < 4; ++db)
#pragma unroll
            for (int r = 0; r < 16; ++r) oacc[db][r] *= alpha;

        // ---- O^T += V^T.P^T ----
#pragma unroll
        for (int db = 0; db < 4; ++db) {
            const char* vrow = lds_v + (db * 32 + qcol) * kVRowBytes + hf * 16;
#pragma unroll
            for (int jj = 0; jj < 4; ++jj) {
                const f16x8 a = *reinterpret_cast<const f16x8*>(vrow + jj * 32);
                oacc[db] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, pb[jj], oacc[db], 0, 0, 0);
            }
        }
    }

    // oacc[db][r] is O[query qcol][d = db*32 + 8*(r/4) + 4*hf + r%4], unnormalised.
    const float l_tot = l_run + __shfl_xor(l_run, 32);
    if (!row_ok) return;
    if (p.num_splits == 1) {
        const float inv = (l_tot == 0.f || l_tot != l_tot) ? 1.f : 1.f / l_tot;
        f16* orow = p.out + ((size_t)node * p.Hq + head) * kHeadDim;
#pragma unroll
        for (int db = 0; db < 4; ++db)
#pragma unroll
            for (int rq = 0; rq < 4; ++rq) {
                f16x4 o;
#pragma unroll
                for (int e = 0; e < 4; ++e) o[e] = (f16)(oacc[db][rq * 4 + e] * inv);
                *reinterpret_cast<f16x4*>(orow + db * 32 + rq * 8 + hf * 4) = o;
            }
    } else {
        const size_t prow = ((size_t)g * p.num_splits + split) * p.rows_pad + R;
        float* op = p.o_part + prow * kHeadDim;
#pragma unroll
        for (int db = 0; db < 4; ++db)
#pragma unroll
            for (int rq = 0; rq < 4; ++rq) {
                f32x4 o;
#pragma unroll
                for (int e = 0; e < 4; ++e) o[e] = oacc[db][rq * 4 + e];
                *reinterpret_cast<f32x4*>(op + db * 32 + rq * 8 + hf * 4) = o;
            }
        if (hf == 0) {
            p.ml_part[prow * 2 + 0] = (m_run == -INFINITY) ? -INFINITY : m_run * p.scale_log2;
            p.ml_part[prow * 2 + 1] = l_tot;
        }
    }
}

// Merge of the split partials: M = max_s m_s, L = sum_s l_s 2^(m_s - M),
// O = sum_s 2^(m_s - M) O_s / L  -- the log-sum-exp merge of
// src/flash_attn/src/flash_fwd_kernel.h:2392-2472 in base-2 form.
// One thread per (packed row, 8 output dims).
__global__ __launch_bounds__(256) void tree_attn_combine_kernel(AttnParams p) {
    const int rows = p.group * p.T;
    const int idx = blockIdx.x * 256 + threadIdx.x;
    const int row_all = idx >> 4;  // over Hkv * rows
    const int dchunk = idx & 15;
    if (row_all >= p.Hkv * rows) return;
    const int g = row_all / rows;
    const int R = row_all % rows;
    const int node = R / p.group;
    const int head = g * p.group + R % p.group;

    float M = -INFINITY;
    for (int s = 0; s < p.num_splits; ++s) {
        const size_t prow = ((size_t)g * p.num_splits + s) * p.rows_pad + R;
        const float l = p.ml_part[prow * 2 + 1];
        if (l > 0.f) M = fmaxf(M, p.ml_part[prow * 2 + 0]);
    }
    float acc[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] = 0.f;
    float L = 0.f;
    for (int s = 0; s < p.num_splits; ++s) {
        const size_t prow = ((size_t)g * p.num_splits + s) * p.rows_pad + R;
        const float l = p.ml_part[prow * 2 + 1];
        if (!(l > 0.f)) continue;  // empty split: its O partial was never meaningful
        const float w = __builtin_amdgcn_exp2f(p.ml_part[prow * 2 + 0] - M);
        L += w * l;
        const f32x4* op = reinterpret_cast<const f32x4*>(p.o_part + prow * kHeadDim + dchunk * 8);
        const f32x4 a = op[0], b = op[1];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            acc[e] += w * a[e];
            acc[4 + e] += w * b[e];
        }
    }
    const float inv = (L == 0.f || L != L) ? 1.f : 1.f / L;
    f16x8 o;
#pragma unroll
    for (int e = 0; e < 8; ++e) o[e] = (f16)(acc[e] * inv);
    *reinterpret_cast<f16x8*>(p.out + ((size_t)node * p.Hq + head) * kHeadDim + dchunk * 8) = o;
}

int choose_splits(int T, int group, int Hkv, int max_kv_len) {
    const int num_mtiles = ceil_div(group * T, kRowsPerWg);
    const int ntiles = ceil_div(max_kv_len, kTileN);
    // Aim for ~one workgroup per CU (256 CUs); every split needs at least one tile.
    int splits = 256 / (num_mtiles * Hkv);
    if (splits < 1) splits = 1;
    if (splits > ntiles) splits = ntiles;
    if (splits > 64) splits = 64;
    return splits;
}

}  // namespace
}  // namespace cpmcu

using namespace cpmcu;

extern "C" size_t cpmcu_tree_attention_workspace_bytes(int T, int Hq, int Hkv, int max_kv_len) {
    if (T <= 0 || Hkv <= 0 || Hq <= 0 || Hq % Hkv) return 0;
    const int group = Hq / Hkv;
    const int num_mtiles = ceil_div(group * T, kRowsPerWg);
    const int rows_pad = num_mtiles * kRowsPerWg;
    // sized for the largest split count the library ever picks, so an override fits too
    const size_t splits = 64;
    return align_up((size_t)Hkv * splits * rows_pad * (kHeadDim + 2) * sizeof(float), 256);
}

extern "C" int cpmcu_tree_attention(const void* q, const void* k_pool, const void* v_pool,
                                    const int32_t* block_table, const int32_t* kv_len, int max_kv_len,
                                    const uint64_t* mask, int mask_words, int T, int Hq, int Hkv,
                                    float scale, void* out, void* workspace, size_t workspace_bytes,
                                    int num_splits_override, void* stream) {
    CPMCU_CHECK_ARG(q && k_pool && v_pool && block_table && kv_len && out, "tree_attention: null pointer argument");
    CPMCU_CHECK_ARG(T >= 1 && T <= kMaxTree, "tree_attention: T=%d outside [1, %d]", T, kMaxTree);
    CPMCU_CHECK_ARG(Hkv >= 1 && Hq >= Hkv && Hq % Hkv == 0, "tree_attention: Hq=%d must be a multiple of Hkv=%d", Hq, Hkv);
    CPMCU_CHECK_ARG(max_kv_len >= T, "tree_attention: max_kv_len=%d < T=%d", max_kv_len, T);
    CPMCU_CHECK_ARG(mask == nullptr || mask_words == ceil_div(T, 64) || (mask_words == 1 && T <= 64),
                    "tree_attention: mask_words=%d does not match T=%d", mask_words, T);
    CPMCU_CHECK_ARG(num_splits_override >= 0 && num_splits_override <= 64, "tree_attention: num_splits_override=%d outside [0, 64]", num_splits_override);
    const int group = Hq / Hkv;
    AttnParams p;
    p.q = (const f16*)q;
    p.k_pool = (const f16*)k_pool;
    p.v_pool = (const f16*)v_pool;
    p.block_table = block_table;
    p.kv_len = kv_len;
    p.mask = mask;
    p.mask_words = mask ? mask_words : 0;
    p.T = T;
    p.Hq = Hq;
    p.Hkv = Hkv;
    p.group = group;
    p.num_mtiles = ceil_div(group * T, kRowsPerWg);
    p.rows_pad = p.num_mtiles * kRowsPerWg;
    p.num_splits = num_splits_override > 0 ? num_splits_override : choose_splits(T, group, Hkv, max_kv_len);
    p.scale_log2 = scale * 1.4426950408889634f;
    p.out = (f16*)out;
    p.o_part = nullptr;
    p.ml_part = nullptr;
    if (p.num_splits > 1) {
        const size_t o_bytes = (size_t)Hkv * p.num_splits * p.rows_pad * kHeadDim * sizeof(float);
        const size_t ml_bytes = (size_t)Hkv * p.num_splits * p.rows_pad * 2 * sizeof(float);
        CPMCU_CHECK_ARG(workspace && workspace_bytes >= o_bytes + ml_bytes,
                        "tree_attention: workspace of %zu bytes needed, %zu given", o_bytes + ml_bytes, workspace_bytes);
        p.o_part = (float*)workspace;
        p.ml_part = (float*)((char*)workspace + o_bytes);
    }
    hipStream_t st = resolve_stream(stream);
    const int nsh = p.num_splits * Hkv;
    const int grid = kXcds * ceil_div(nsh, kXcds) * p.num_mtiles;
    hipLaunchKernelGGL(tree_attn_split_kernel, dim3(grid), dim3(kThreads), 0, st, p);
    CPMCU_LAUNCH_CHECK();
    if (p.num_splits > 1) {
        const int threads_total = Hkv * group * T * 16;
        hipLaunchKernelGGL(tree_attn_combine_kernel, dim3(ceil_div(threads_total, 256)), dim3(256), 0, st, p);
        CPMCU_LAUNCH_CHECK();
    }
    return CPMCU_OK;
}
