// Exact top-k, log-softmax, FR-Spec id map-back and row gather for gfx950.
//
// Ordering contract of the reference's bitonic TopK (src/model/topk.cuh:17): value descending,
// equal values -> lower index first.  Here every element becomes one 64-bit key
//   (order-preserving 16-bit image of the fp16 value) << 32 | (0xFFFFFFFF - index)
// so "largest key first" IS that ordering and keys are unique -- no sorting network, no padding to
// powers of two, any k.  Two ways to the k largest keys:
//   * topk_row_kernel, one launch: rows of up to 32768 values (the FR-Spec vocabulary) stay in the
//     registers of one workgroup, which bounds the k-th value from its waves' lane maxima, compacts the
//     few candidates above the bound and ranks them by counting;
//   * topk_chunk_kernel + topk_merge_kernel: longer rows, k rounds of a workgroup-wide maximum per
//     2048-element chunk and again over the chunks' winners.
//
// FR-Spec fusion: the draft head ranks log-probabilities that were rounded to fp16 BEFORE
// ranking (src/model/eagle.cuh:87), so rounding ties must be reproduced exactly.  The kernels
// therefore recompute f16((z - max) - ln sum) from the fp16 logits and the row statistics
// reduced from the GEMM's per-workgroup partials, and rank that.
#include "common.h"
#include "internal.h"
#include "timeline.h"
#include "topk_keys.h"

namespace cpmcu {
namespace {

// Timeline records of the row kernel (timeline.h): 0 start, 1 the row is in registers as ordered images, 2 bound and row
// statistics known, 3 candidate lanes handed to LDS, 4 candidates extracted, 5 ranked, 6 outputs written.
CPMCU_TIMELINE_STORAGE(g_topk_timeline)

struct TopkParams {
    const uint16_t* x;  // [n][dim] fp16 bits
    int n, dim, top, nchunks;
    int slice_len;      // row kernel: elements per workgroup when a row is cut into slices (0: the whole row)
    int ragged;         // row kernel: rows are not whole 16-byte pieces (dim not a multiple of 8, or x not 16-byte aligned)
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

// E: the element type of the values (it matters only with the fused log-softmax, which does arithmetic on them; the raw
// ranking works on bit patterns whose order is the same for both types).  The kernels proper are thin wrappers below.
template <bool LOGSOFTMAX, typename E>
__device__ __forceinline__ void topk_chunk_body(const TopkParams& p) {
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
                const float z = Elem<E>::from_bits(bits);
                bits = Elem<E>::to_bits((z - m) - lse);  // src/model/eagle.cuh:87
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
__global__ __launch_bounds__(kTopkThreads) void topk_chunk_kernel(TopkParams p) { topk_chunk_body<LOGSOFTMAX, f16>(p); }
__global__ __launch_bounds__(kTopkThreads) void topk_chunk_bf16_kernel(TopkParams p) { topk_chunk_body<true, bf16>(p); }

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

// One-launch top-k for rows of at most kRowMaxDim elements: one 1024-thread workgroup per row keeps
// the whole row in registers, two values per register as order-preserving 16-bit images of the raw
// input ("raw images": bits ^ (sign ? 0xFFFF : 0x8000); -0 is one below +0 here, which every bound
// below allows for).
//   1. a lower bound of the k-th largest value: every wave takes the k-th largest of its 64
//      per-lane maxima (bisection over the 16 bits with ballots, no barrier); the largest of the 16
//      wave results has at least k elements at or above it, and on anything but tie-heavy data only
//      a few hundred.  Beyond k = 16 that bound sinks towards the smallest lane maximum, so the waves whose 64 lanes all
//      hold elements also take their ceil(k / waves)-th largest lane maximum each: the smallest of those has k lanes at
//      or above it as well, and the higher of the two bounds is used (k up to 128);
//   2. fused log-softmax: ranking is on f16((z - max) - ln sum), a monotone map of z that merges
//      neighbours, so the bound moves down by four ulps of the mapped bound -- every z that can map
//      to the same fp16 value or above stays a candidate -- and only candidates are mapped;
//   3. candidates go to LDS as exact 64-bit keys; each counts the candidates with a larger key:
//      that count IS its output slot.
// More than kRowCap candidates (rows dominated by one value): k rounds of a workgroup-wide maximum
// over the register-resident values instead, each round taking the largest key below the previous winner.
constexpr int kRowThreads = 1024;
constexpr int kRowWaves = kRowThreads / 64;
constexpr int kRowPieces = 4;                          // 16-byte pieces per thread
constexpr int kRowElems = kRowPieces * 8;
constexpr int kRowMaxDim = kRowThreads * kRowElems;    // 32768
constexpr int kRowCap = kRowThreads;                   // candidate keys held in LDS
constexpr int kRowBoundDrop = 4;                       // low bits of the bound that are not searched
constexpr int kRowDenseWaves = 8;                      // waves that extract the candidates
constexpr int kRowLaneCap = 512;                       // threads with candidates whose registers LDS can take
constexpr int kRowMaxTop = 128;                        // output slots are ranks below k <= kRowCap; beyond 64 see row_kernel_ranks()

typedef int16_t s16x2 __attribute__((ext_vector_type(2)));
typedef uint16_t u16x2 __attribute__((ext_vector_type(2)));

template <bool LOGSOFTMAX, typename E>
__device__ __forceinline__ void topk_row_body(const TopkParams& p) {
    __shared__ __attribute__((aligned(16))) uint64_t cand[kRowCap];
    __shared__ int rank[kRowCap];
    __shared__ uint64_t wave_best[2][kRowWaves];
    __shared__ float row_m_lse[2];
    __shared__ uint32_t wave_kth[kRowWaves], wave_few[kRowWaves];
    __shared__ int ncand, nlanes;
    __shared__ uint4 lanebuf[kRowPieces][kRowLaneCap];  // piece-major: neighbouring slots are neighbouring 16 bytes
    __shared__ int lane_owner[kRowLaneCap];
    CPMCU_STAMP(g_topk_timeline, blockIdx.x, 0);
    const int row = blockIdx.x;
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    // a row longer than kRowMaxDim is cut into slices, one workgroup each: this one ranks elements [slice_base, slice_base + len) and
    // leaves its k best as keys for the merge launch instead of writing the outputs
    const bool sliced = p.slice_len != 0;
    const int slice_base = sliced ? blockIdx.y * p.slice_len : 0;
    const int len = sliced ? min(p.slice_len, p.dim - slice_base) : p.dim;
    const int npieces = (len + 7) >> 3;
    const uint4* xr = (const uint4*)(p.x + (size_t)row * p.dim + slice_base);
    uint64_t* slice_out = sliced ? p.cand + ((size_t)row * gridDim.y + blockIdx.y) * p.top : nullptr;
    if (sliced && tid < p.top) slice_out[tid] = 0;  // slots this slice cannot fill stay empty (overwritten behind a barrier)
    // slots beyond the row read as 0xFFFF, whose raw image is 0: below every bound that is used
    uint4 raw[kRowPieces];
    if (!p.ragged) {
#pragma unroll
        for (int j = 0; j < kRowPieces; ++j) {
            const int pc = j * kRowThreads + tid;
            raw[j] = pc < npieces ? xr[pc] : make_uint4(~0u, ~0u, ~0u, ~0u);
        }
    } else {
        // rows that do not start on 16 bytes or do not end on a whole piece: element by element
        const uint16_t* xe = (const uint16_t*)xr;
#pragma unroll
        for (int j = 0; j < kRowPieces; ++j) {
            const int e0 = (j * kRowThreads + tid) * 8;
            uint32_t w4[4];
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const uint32_t a = e0 + 2 * q < len ? xe[e0 + 2 * q] : 0xFFFFu;
                const uint32_t b = e0 + 2 * q + 1 < len ? xe[e0 + 2 * q + 1] : 0xFFFFu;
                w4[q] = a | (b << 16);
            }
            raw[j] = make_uint4(w4[0], w4[1], w4[2], w4[3]);
        }
    }
    if (tid == 0) {
        ncand = 0;
        nlanes = 0;
    }
    rank[tid] = 0;
    cand[tid] = 0;
    // row statistics from the GEMM's per-workgroup (max, sum exp(z - max)) partials, on wave 0: the
    // first 256 partials are requested here and reduced after the bound search, whose instructions
    // cover their latency
    float pa[4], pb[4];
    if (LOGSOFTMAX && wave == 0) {
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int c = lane + u * 64;
            pa[u] = c < p.grid ? p.part_max[(size_t)c * p.stride + row] : -INFINITY;
            pb[u] = c < p.grid ? p.part_sum[(size_t)c * p.stride + row] : 0.f;
        }
    }
    // raw images, two per register
    uint32_t img[kRowElems / 2];
    u16x2 lmax2 = {0, 0};
#pragma unroll
    for (int j = 0; j < kRowPieces; ++j) {
        const uint32_t w4[4] = {raw[j].x, raw[j].y, raw[j].z, raw[j].w};
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const s16x2 sx = __builtin_bit_cast(s16x2, w4[q]);
            const uint32_t sign = __builtin_bit_cast(uint32_t, sx >> 15);
            const uint32_t o = w4[q] ^ (sign | 0x80008000u);
            img[j * 4 + q] = o;
            lmax2 = __builtin_elementwise_max(lmax2, __builtin_bit_cast(u16x2, o));
        }
    }
    const uint32_t lmax = lmax2[0] > lmax2[1] ? lmax2[0] : lmax2[1];
#ifdef CPMCU_TIMELINE
    asm volatile("" ::"v"(lmax));
#endif
    CPMCU_STAMP(g_topk_timeline, blockIdx.x, 1);
    // k-th largest of this wave's lane maxima, rounded down to a multiple of 2^kRowBoundDrop (0 when
    // fewer than k lanes hold anything): a slightly lower bound is as valid and costs fewer steps
    // (with fused statistics wave 0 reduces those meanwhile and contributes no bound: any subset of
    // the waves gives a valid one)
    uint32_t kth = 0;
    // k > 16: the full waves share k between them (wave 0 is busy with the statistics when those are fused)
    const int first_wave = LOGSOFTMAX ? 1 : 0;
    const int full_waves = min(kRowWaves, npieces >> 6);
    // (bfloat16 rows tie so often that the shared bound pays at every k: 6.0 against 6.4 us for the top 10 of 32768; fp16: 5.9 either way)
    const bool spread = (p.top > 16 || !std::is_same<E, f16>::value) && full_waves - first_wave >= 2;
    if (!(LOGSOFTMAX && wave == 0)) {
        for (int bit = 15; bit >= kRowBoundDrop; --bit) {
            const uint32_t c = kth | (1u << bit);
            if (__popcll(__ballot(lmax >= c)) >= p.top) kth = c;
        }
        if (spread && wave < full_waves) {
            const int few = (p.top + full_waves - first_wave - 1) / (full_waves - first_wave);
            uint32_t kf = 0;
            if (few == 1) {
                kf = wave_reduce_b32(lmax, [](uint32_t a, uint32_t b) { return a > b ? a : b; });
            } else {
                for (int bit = 15; bit >= kRowBoundDrop; --bit) {
                    const uint32_t c = kf | (1u << bit);
                    if (__popcll(__ballot(lmax >= c)) >= few) kf = c;
                }
            }
            if (lane == 0) wave_few[wave] = kf;
        }
    }
    if (lane == 0) wave_kth[wave] = kth;
    if (LOGSOFTMAX && wave == 0) {
        float a = -INFINITY, b = 0.f;
        for (int c0 = lane;;) {
            const float mm = fmaxf(fmaxf(a, fmaxf(pa[0], pa[1])), fmaxf(pa[2], pa[3]));
            float acc = (a == -INFINITY) ? 0.f : b * __expf(a - mm);
#pragma unroll
            for (int u = 0; u < 4; ++u) acc += (pa[u] == -INFINITY) ? 0.f : pb[u] * __expf(pa[u] - mm);
            a = mm;
            b = acc;
            c0 += 256;
            if (c0 - lane >= p.grid) break;
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int c = c0 + u * 64;
                pa[u] = c < p.grid ? p.part_max[(size_t)c * p.stride + row] : -INFINITY;
                pb[u] = c < p.grid ? p.part_sum[(size_t)c * p.stride + row] : 0.f;
            }
        }
        const float wm = wave_max_f32(a);
        b = wave_sum_f32((a == -INFINITY) ? 0.f : b * __expf(a - wm));
        if (lane == 0) {
            const float l = __logf(b);
            row_m_lse[0] = wm;
            row_m_lse[1] = l;
            if (p.row_stats && slice_base == 0) {
                p.row_stats[row * 2 + 0] = wm;
                p.row_stats[row * 2 + 1] = l;
            }
        }
    }
    __syncthreads();
    CPMCU_STAMP(g_topk_timeline, blockIdx.x, 2);
    uint32_t bound = wave_kth[0];
#pragma unroll
    for (int w = 1; w < kRowWaves; ++w) bound = wave_kth[w] > bound ? wave_kth[w] : bound;
    if (spread) {
        uint32_t least = ~0u;
#pragma unroll
        for (int w = 0; w < kRowWaves; ++w)
            if (w >= first_wave && w < full_waves) least = wave_few[w] < least ? wave_few[w] : least;
        bound = least > bound ? least : bound;
    }
    uint32_t lo = bound > 0 ? bound - 1 : 0;  // candidates: raw image >= lo
    float m = 0.f, lse = 0.f;
    if (LOGSOFTMAX) {
        m = row_m_lse[0];
        lse = row_m_lse[1];
        if (bound > 0) lo = mapped_lower_image<E>(bound, m, lse);
    }
    // a row that fits the candidate buffer needs no bound: every element whose image is not 0 is a candidate (image 0 is
    // the NaN 0xFFFF, which also pads the registers beyond the row; a row that holds one goes the way of the k rounds below)
    if (lo == 0 && !sliced && p.dim <= kRowCap) lo = 1;

    const auto key_from_image = [&](uint32_t o, int idx) -> uint64_t {
        uint16_t bits = (uint16_t)((o & 0x8000u) ? (o ^ 0x8000u) : (o ^ 0xFFFFu));
        if (LOGSOFTMAX) {
            const float z = Elem<E>::from_bits(bits);
            bits = Elem<E>::to_bits((z - m) - lse);  // src/model/eagle.cuh:87
        }
        return make_key(bits, idx);
    };
    // threads holding anything at or above the bound hand their 16 registers to LDS ...
    const bool bounded = lo != 0;
    if (bounded && lmax >= lo) {
        const int s = atomicAdd(&nlanes, 1);
        if (s < kRowLaneCap) {
#pragma unroll
            for (int j = 0; j < kRowPieces; ++j) lanebuf[j][s] = make_uint4(img[4 * j], img[4 * j + 1], img[4 * j + 2], img[4 * j + 3]);
            lane_owner[s] = tid;
        }
    }
    __syncthreads();
    CPMCU_STAMP(g_topk_timeline, blockIdx.x, 3);
    const int NT = nlanes;
    const bool compact = bounded && NT <= kRowLaneCap;
    // ... where a few waves take them over with most of their lanes busy: bit mask of the
    // elements at or above the bound (saturating packed subtract: non-zero half <=> image >= lo),
    // one exact 64-bit key per element
    if (compact && wave < kRowDenseWaves) {
        const u16x2 below = __builtin_bit_cast(u16x2, (lo - 1) * 0x10001u);
        const u16x2 one2 = {1, 1};
        const int per_wave = (NT + kRowDenseWaves - 1) / kRowDenseWaves;
        for (int i = lane; i < per_wave; i += 64) {
            const int s = wave * per_wave + i;
            if (s >= NT) break;
            // bit r: low half of register r is a candidate, bit 16 + r: its high half
            uint32_t em = 0;
#pragma unroll
            for (int j = 0; j < kRowPieces; ++j) {
                const uint4 v = lanebuf[j][s];
                const uint32_t w4[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const u16x2 d = __builtin_elementwise_sub_sat(__builtin_bit_cast(u16x2, w4[q]), below);
                    em |= __builtin_bit_cast(uint32_t, __builtin_elementwise_min(d, one2)) << (4 * j + q);
                }
            }
            const int owner = lane_owner[s];
            // slots: prefix sum of the per-lane counts over the wave, one bit plane of the counts at a
            // time, and one atomic by the first active lane
            const int n = __popc(em);
            const uint64_t lanes_below = (1ull << lane) - 1ull;
            int before = 0, total = 0;
            for (int bit = 0; __ballot((n >> bit) != 0) != 0; ++bit) {
                const uint64_t plane = __ballot((n >> bit) & 1);
                before += __popcll(plane & lanes_below) << bit;
                total += __popcll(plane) << bit;
            }
            int base = 0;
            if (lane == __builtin_ctzll(__ballot(true))) base = atomicAdd(&ncand, total);
            int slot = __builtin_amdgcn_readfirstlane(base) + before;
            while (em) {
                const int t = __builtin_ctz(em);
                em &= em - 1;
                const int e = 2 * (t & 15) + (t >> 4);  // element of the owner thread
                const uint32_t o = ((const uint16_t*)&lanebuf[e >> 3][s])[e & 7];
                if (slot < kRowCap) cand[slot] = key_from_image(o, slice_base + ((e >> 3) * kRowThreads + owner) * 8 + (e & 7));
                ++slot;
            }
        }
    }
    __syncthreads();
    CPMCU_STAMP(g_topk_timeline, blockIdx.x, 4);
    const int C = ncand;
    if (compact && C <= kRowCap && C >= p.top) {
        int shift = 6;
        while ((1 << shift) < C) ++shift;
        const int i = tid & ((1 << shift) - 1);
        const int part = tid >> shift, nparts = kRowThreads >> shift;
        // the mapped id of candidate tid is fetched now and used after the ranking
        int32_t mapped = 0;
        if (tid < C && p.ids && !sliced) mapped = p.remap ? p.remap[key_index(cand[tid])] : key_index(cand[tid]);
        if (i < C) {
            // slots from C on hold key 0, so whole groups of eight can be compared
            const uint64_t my = cand[i];
            const int chunk = ((C + nparts - 1) / nparts + 7) & ~7;
            int r = 0;
            for (int j = part * chunk; j < (part + 1) * chunk; j += 8) {
                uint64_t o[8];
#pragma unroll
                for (int u = 0; u < 8; ++u) o[u] = cand[j + u];
#pragma unroll
                for (int u = 0; u < 8; ++u) r += o[u] > my ? 1 : 0;
            }
            if (r) atomicAdd(&rank[i], r);
        }
        __syncthreads();
        CPMCU_STAMP(g_topk_timeline, blockIdx.x, 5);
        if (tid < C && rank[tid] < p.top) {
            const uint64_t key = cand[tid];
            if (sliced) {
                slice_out[rank[tid]] = key;
            } else {
                const int idx = key_index(key);
                const size_t o = (size_t)row * p.top + rank[tid];
                p.val[o] = LOGSOFTMAX ? key_bits(key) : p.x[(size_t)row * p.dim + idx];
                p.pos[o] = idx;
                if (p.ids) p.ids[o] = mapped;
            }
        }
        CPMCU_STAMP(g_topk_timeline, blockIdx.x, 6);
        return;
    }
    uint64_t prev = ~0ull;
    for (int round = 0; round < p.top; ++round) {
        uint64_t mine = 0;
#pragma unroll
        for (int j = 0; j < kRowPieces; ++j) {
            const int e0 = (j * kRowThreads + tid) * 8;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const uint32_t o = (img[j * 4 + (e >> 1)] >> ((e & 1) * 16)) & 0xFFFFu;
                const uint64_t key = e0 + e < len ? key_from_image(o, slice_base + e0 + e) : 0ull;
                if (key < prev && key > mine) mine = key;
            }
        }
        const uint64_t wbest = wave_max_u64(mine);
        uint64_t* wb = wave_best[round & 1];
        if (lane == 0) wb[wave] = wbest;
        __syncthreads();
        uint64_t best = wb[0];
#pragma unroll
        for (int w = 1; w < kRowWaves; ++w) best = wb[w] > best ? wb[w] : best;
        if (tid == 0) {
            if (sliced) slice_out[round] = best;
            else emit_final<LOGSOFTMAX>(p, row, round, best);
        }
        prev = best;
        if (best == 0) break;
    }
}

// The slices' k best keys of a row (at most kSliceMergeCap of them, empty slots are 0) ranked by counting: one workgroup per
// row, the count of larger keys is the output slot.
constexpr int kSliceMergeCap = 1024;
template <bool LOGSOFTMAX>
__global__ __launch_bounds__(kTopkThreads) void topk_slice_merge_kernel(TopkParams p) {
    __shared__ uint64_t keys[kSliceMergeCap];
    const int row = blockIdx.x;
    const int ncand = p.nchunks * p.top;
    const uint64_t* in = p.cand + (size_t)row * ncand;
    for (int i = threadIdx.x; i < ncand; i += kTopkThreads) keys[i] = in[i];
    __syncthreads();
    for (int i = threadIdx.x; i < ncand; i += kTopkThreads) {
        const uint64_t my = keys[i];
        if (my == 0) continue;
        int r = 0;
        for (int j = 0; j < ncand; ++j) r += keys[j] > my ? 1 : 0;
        if (r < p.top) emit_final<LOGSOFTMAX>(p, row, r, my);
    }
}

template <bool LOGSOFTMAX>
__global__ __launch_bounds__(kRowThreads) void topk_row_kernel(TopkParams p) { topk_row_body<LOGSOFTMAX, f16>(p); }
__global__ __launch_bounds__(kRowThreads) void topk_row_bf16_kernel(TopkParams p) { topk_row_body<true, bf16>(p); }

// log_softmax in place (src/model/eagle.cuh:29-89): one workgroup per row.  The row is walked in 16-byte pieces from its
// first 16-byte boundary on; the first four pieces of every thread stay in registers between the three passes (maximum, sum,
// write), so a row of up to 32768 elements is read once; the up to seven elements in front of the first piece and behind
// the last go one to a thread.
template <typename E>
__device__ __forceinline__ void log_softmax_body(uint16_t* x, int dim, float* row_stats) {
    __shared__ float red[16];
    constexpr int kKeep = 4;
    const int row = blockIdx.x;
    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    uint16_t* xr = x + (size_t)row * dim;
    const int head = min(dim, (int)(((16 - ((uintptr_t)xr & 15)) & 15) >> 1));
    const int npieces = (dim - head) >> 3;
    const int tail0 = head + npieces * 8, ntail = dim - tail0;
    uint4* xp = (uint4*)(xr + head);
    const int single = tid < head ? tid : tid < head + ntail ? tail0 + (tid - head) : -1;  // this thread's element outside the pieces
    const float single_v = single >= 0 ? Elem<E>::from_bits(xr[single]) : -INFINITY;
    const uint32_t ninf2 = Elem<E>::to_bits(-INFINITY) * 0x10001u;
    uint4 keep[kKeep];
#pragma unroll
    for (int j = 0; j < kKeep; ++j) {
        const int pc = j * 1024 + tid;
        keep[j] = pc < npieces ? xp[pc] : make_uint4(ninf2, ninf2, ninf2, ninf2);
    }
    const auto lo = [](uint32_t w) { return Elem<E>::from_bits((uint16_t)(w & 0xFFFFu)); };
    const auto hi = [](uint32_t w) { return Elem<E>::from_bits((uint16_t)(w >> 16)); };
    const auto piece_max = [&](const uint4& v, float a) {
        a = fmaxf(fmaxf(a, lo(v.x)), fmaxf(hi(v.x), lo(v.y)));
        a = fmaxf(fmaxf(a, hi(v.y)), fmaxf(lo(v.z), hi(v.z)));
        return fmaxf(a, fmaxf(lo(v.w), hi(v.w)));
    };
    float m = single_v;
#pragma unroll
    for (int j = 0; j < kKeep; ++j) m = piece_max(keep[j], m);
    for (int pc = kKeep * 1024 + tid; pc < npieces; pc += 1024) m = piece_max(xp[pc], m);
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) m = fmaxf(m, __shfl_xor(m, off));
    if (lane == 0) red[wave] = m;
    __syncthreads();
    m = red[0];
#pragma unroll
    for (int w = 1; w < 16; ++w) m = fmaxf(m, red[w]);
    __syncthreads();
    const auto piece_sum = [&](const uint4& v, float a) {
        a += expf(lo(v.x) - m) + expf(hi(v.x) - m);
        a += expf(lo(v.y) - m) + expf(hi(v.y) - m);
        a += expf(lo(v.z) - m) + expf(hi(v.z) - m);
        return a + (expf(lo(v.w) - m) + expf(hi(v.w) - m));
    };
    float s = single >= 0 ? expf(single_v - m) : 0.f;
#pragma unroll
    for (int j = 0; j < kKeep; ++j)
        if (j * 1024 + tid < npieces) s = piece_sum(keep[j], s);
    for (int pc = kKeep * 1024 + tid; pc < npieces; pc += 1024) s = piece_sum(xp[pc], s);
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) s += __shfl_xor(s, off);
    if (lane == 0) red[wave] = s;
    __syncthreads();
    s = 0.f;
#pragma unroll
    for (int w = 0; w < 16; ++w) s += red[w];
    const float lse = logf(s);
    const auto map2 = [&](uint32_t w) {
        return (uint32_t)Elem<E>::to_bits((lo(w) - m) - lse) | ((uint32_t)Elem<E>::to_bits((hi(w) - m) - lse) << 16);  // src/model/eagle.cuh:87
    };
    const auto piece_map = [&](const uint4& v) { return make_uint4(map2(v.x), map2(v.y), map2(v.z), map2(v.w)); };
#pragma unroll
    for (int j = 0; j < kKeep; ++j)
        if (j * 1024 + tid < npieces) xp[j * 1024 + tid] = piece_map(keep[j]);
    for (int pc = kKeep * 1024 + tid; pc < npieces; pc += 1024) xp[pc] = piece_map(xp[pc]);
    if (single >= 0) xr[single] = Elem<E>::to_bits((single_v - m) - lse);
    if (tid == 0 && row_stats) {
        row_stats[row * 2 + 0] = m;
        row_stats[row * 2 + 1] = lse;
    }
}

__global__ __launch_bounds__(1024) void log_softmax_kernel(uint16_t* x, int dim, float* row_stats) { log_softmax_body<f16>(x, dim, row_stats); }
__global__ __launch_bounds__(1024) void log_softmax_bf16_kernel(uint16_t* x, int dim, float* row_stats) { log_softmax_body<bf16>(x, dim, row_stats); }

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

// Whether the row kernel finds a bound for the k-th largest of a row of `dim` elements (else it would fall to its k rounds):
// up to 64 any wave's lanes do; beyond, the waves that are full of elements share k, at most 64 lanes' worth each.
static bool row_kernel_ranks(int dim, int top, bool fused_stats) {
    if (top <= 64 || dim <= kRowCap) return top <= kRowMaxTop;
    const int sharing = std::min(kRowWaves, dim / 8 / 64) - (fused_stats ? 1 : 0);
    return top <= kRowMaxTop && sharing >= 2 && sharing * 64 >= top;
}

int launch_topk(const void* x, int n, int dim, int top, void* val, int32_t* pos, int32_t* ids,
                const int32_t* token_id_remap, const TopkStatsSource* stats, void* workspace,
                size_t workspace_bytes, hipStream_t st) {
    TopkParams p;
    p.x = (const uint16_t*)x;
    p.n = n;
    p.dim = dim;
    p.top = top;
    p.nchunks = ceil_div(dim, kChunk);
    p.slice_len = 0;
    p.ragged = dim % 8 != 0 || ((uintptr_t)x & 15) != 0;
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
    // rows that fit one workgroup's registers: one launch, no candidate buffer
    const bool row_kernel = options().topk_row_kernel != 0;
    if (row_kernel && dim <= kRowMaxDim && row_kernel_ranks(dim, top, stats != nullptr)) {
        if (stats && options().dtype == 1) hipLaunchKernelGGL(topk_row_bf16_kernel, dim3(n), dim3(kRowThreads), 0, st, p);
        else if (stats) hipLaunchKernelGGL(topk_row_kernel<true>, dim3(n), dim3(kRowThreads), 0, st, p);
        else hipLaunchKernelGGL(topk_row_kernel<false>, dim3(n), dim3(kRowThreads), 0, st, p);
        CPMCU_LAUNCH_CHECK();
        return CPMCU_OK;
    }
    // longer rows in slices of at most kRowMaxDim elements: the row kernel on every slice, and a merge of the slices' k best
    const int nslices = ceil_div(dim, kRowMaxDim);
    if (row_kernel && top <= kRowMaxTop && nslices * top <= kSliceMergeCap && workspace &&
        workspace_bytes >= (size_t)n * nslices * top * sizeof(uint64_t)) {
        p.slice_len = (ceil_div(dim, nslices) + 7) / 8 * 8;
        p.nchunks = nslices;
        const dim3 grid(n, nslices);
        if (stats && options().dtype == 1) hipLaunchKernelGGL(topk_row_bf16_kernel, grid, dim3(kRowThreads), 0, st, p);
        else if (stats) hipLaunchKernelGGL(topk_row_kernel<true>, grid, dim3(kRowThreads), 0, st, p);
        else hipLaunchKernelGGL(topk_row_kernel<false>, grid, dim3(kRowThreads), 0, st, p);
        CPMCU_LAUNCH_CHECK();
        if (stats) hipLaunchKernelGGL(topk_slice_merge_kernel<true>, dim3(n), dim3(kTopkThreads), 0, st, p);
        else hipLaunchKernelGGL(topk_slice_merge_kernel<false>, dim3(n), dim3(kTopkThreads), 0, st, p);
        CPMCU_LAUNCH_CHECK();
        return CPMCU_OK;
    }
    CPMCU_CHECK_ARG(p.nchunks * top <= kMaxCand, "topk: dim=%d with top=%d needs %d merge candidates, limit %d",
                    dim, top, p.nchunks * top, kMaxCand);
    if (p.nchunks > 1) {
        const size_t need = (size_t)n * p.nchunks * top * sizeof(uint64_t);
        CPMCU_CHECK_ARG(workspace && workspace_bytes >= need, "topk: workspace of %zu bytes needed, %zu given", need, workspace_bytes);
    }
    const dim3 grid(p.nchunks, n);
    if (stats) {
        if (options().dtype == 1) hipLaunchKernelGGL(topk_chunk_bf16_kernel, grid, dim3(kTopkThreads), 0, st, p);
        else hipLaunchKernelGGL(topk_chunk_kernel<true>, grid, dim3(kTopkThreads), 0, st, p);
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
    if (options().dtype == 1) hipLaunchKernelGGL(log_softmax_bf16_kernel, dim3(n), dim3(1024), 0, resolve_stream(stream), (uint16_t*)x, dim, row_stats);
    else hipLaunchKernelGGL(log_softmax_kernel, dim3(n), dim3(1024), 0, resolve_stream(stream), (uint16_t*)x, dim, row_stats);
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
    bool fused = false;
    int rc0 = launch_frspec_fused(hidden, w, w_layout, token_id_remap, n, V, H, k, logits, row_stats, topk_val, topk_pos, topk_ids, workspace,
                                  st, &fused);
    if (rc0 != CPMCU_OK || fused) return rc0;
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

// 1: a call of cpmcu_frspec_head_topk with this shape on this workspace runs as one launch (and a publication state of
// the library is now assigned to the pair, if it had none); 0: as GEMM launch + top-k launch.
extern "C" int cpmcu_frspec_head_mode(const void* workspace, int w_layout, int n, int V, int H, int k) {
    if (workspace == nullptr || n < 1 || n > 16 || k < 1 || V < 1 || H < 1) return 0;
    bool fused = false;
    // the planning needs a non-null, 8-byte aligned logits pointer only to check alignment
    if (launch_frspec_fused(workspace, workspace, w_layout, nullptr, n, V, H, k, (void*)workspace, nullptr, nullptr, nullptr, nullptr, workspace,
                            nullptr, &fused, true) != CPMCU_OK)
        return 0;
    return fused ? 1 : 0;
}

// Gives back the library-side states of a head workspace that is about to be freed (no launch on it in flight or captured).
extern "C" int cpmcu_head_release_workspace(const void* workspace) {
    CPMCU_CHECK_ARG(workspace, "head_release_workspace: null pointer argument");
    head_fuse_release_workspace(workspace);
    return CPMCU_OK;
}

CPMCU_TIMELINE_READER(cpmcu_timeline_read_topk, cpmcu::g_topk_timeline)
