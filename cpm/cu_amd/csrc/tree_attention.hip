// Tree-verify flash attention for gfx950 (MI355X): tree-masked draft queries
// against the paged prefix KV plus the in-tree KV, GQA-packed, fp16 MFMA with
// fp32 accumulation, split over the KV stream; the split workgroups merge their
// partial results themselves (a second kernel does it for launches that do not
// fit the GPU's CUs or have more than 32 splits).
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
//  * K/V tiles (64 keys, 32 KB) go HBM/L2 -> LDS with direct-to-LDS loads
//    (global_load_lds_dwordx4) into a 4-stage ring, XOR-swizzled through the
//    choice of the global address each lane fetches, so no registers are spent
//    on staging and two tiles are always in flight behind the two being
//    consumed.
//  * A workgroup is 8 waves.  For short contexts they are 2 KV groups x 4 row
//    waves over the same 128 packed rows: the groups take alternate tiles of
//    the ring and are merged through LDS at the end -- half the partial traffic
//    of splitting the same work over two workgroups.  For long contexts they
//    are 8 row waves over 256 packed rows, every tile feeding all of them.
//  * The Q rows and the tree mask reach the registers through LDS (whole rows,
//    coalesced), not through per-lane fetches in the MFMA operand layout.
//  * Workgroups are mapped so that all M-tiles that stream the same KV range
//    land on the same XCD (workgroup id modulo 8) and share its L2.
#include "common.h"
#include "internal.h"
#include "timeline.h"

#include <map>
#include <mutex>
#include <type_traits>
#include <algorithm>
#include <utility>
#include <vector>

namespace cpmcu {
namespace {

constexpr int kTileN = 64;                  // keys per LDS tile
constexpr int kWaves = 8;                   // waves per workgroup = KV groups x row waves
constexpr int kRowsPerWave = 32;            // packed query rows per wave (one MFMA N block)
constexpr int kThreads = kWaves * 64;
// The kernel comes in two shapes (template parameter G = KV groups per workgroup):
//   G = 2: 4 row waves (128 packed rows) x 2 KV groups that take alternate tiles and are merged through
//          LDS at the end.  More (KV head, M-tile) units, so fewer splits fill the GPU: short contexts.
//   G = 1: 8 row waves (256 packed rows) on every tile.  Each tile fetched feeds twice the rows and
//          three tiles are in flight behind the one being consumed: long contexts.
constexpr int rows_per_wg(int G) { return (kWaves / G) * kRowsPerWave; }
constexpr int kStages = 4;
constexpr int kKTileBytes = kTileN * kHeadDim * 2;  // 16 KB, row = one key (256 B)
constexpr int kVTileBytes = kHeadDim * kTileN * 2;  // 16 KB, row = one dim (128 B)
constexpr int kStageBytes = kKTileBytes + kVTileBytes;
constexpr int kVStageRows = 64;  // appended V rows staged in LDS ahead of their transposition
constexpr int kMaxSplits = 128;
constexpr int kMergeMaxSplits = 32;  // most splits of a launch that merges its own partials: arrivals on one counter
                                     // serialise, about 0.15 us each
constexpr int kXcds = 8;
constexpr float kLazyLog2 = 8.f;  // slack of the lazily updated softmax reference, in log2 units

typedef __attribute__((address_space(3))) void* lds_ptr_t;

// Set by a launch whose device-side length does not fit what the host promised (above max_kv_len, or shorter
// than the query rows / the masked range): the launch then works on the length clamped into that range -- every
// access stays inside the page table -- and this word keeps the offending length for the next synchronising call.
// `abandoned` counts merge waits that ran out (see the merge inside the launch below): workgroups that left their share to
// the last arrival of their unit (the output was complete, only late).
struct AttnReport {
    int bad_length;
    unsigned int abandoned;
};
__device__ AttnReport g_attn_report;

// Timeline records of the split kernel (timeline.h; kept in registers and stored at the end, since the kernel counts its
// outstanding memory operations by hand): 0 start, 1 K loop entered, 2 K loop left, 3 KV groups merged, 4 partials
// issued, 5 partials acknowledged, 6 every split of the unit has arrived, 7 end; notes: 8 iterations, 9 tiles, 10 split,
// 11 M-tile; 12 / 13 second / third iteration entered, 14 / 15 last patch of landed tiles (appended rows, end of the
// stream) begun / done.
CPMCU_TIMELINE_STORAGE(g_attn_timeline)

struct AttnParams {
    const f16* q;
    const f16* k_pool;
    const f16* v_pool;
    const int32_t* block_table;
    const int32_t* kv_len;
    const f16* k_new;  // [T][Hkv][128] rows of the tree nodes to append, or null: already in the cache
    const f16* v_new;
    const float2* rope;  // [T][64] (cos, sin) of the tree rows' positions, or null: q and k_new come rotated
    f16* k_pool_w;     // writable aliases of the pools (used only when k_new is set)
    f16* v_pool_w;
    const uint64_t* mask;
    int mask_words;
    int mask_k_range;  // trailing key columns the mask bits refer to (>= T; = T for the verify tree)
    int T, Hq, Hkv, group;
    int group_shift, hkv_shift;  // log2 of group / Hkv when they are powers of two (the usual case), else -1: plain division
    int num_splits, num_mtiles, rows_pad;
    int ntiles_max;  // tiles the split partition spans: ceil(max_kv_len / 64), fixed by the host-side bound
                     // (with a window: the most tiles a window can hold, counted from its first tile)
    int table_pages;    // entries of block_table the caller guarantees: ceil(max_kv_len / 256)
    int max_kv_len;     // the host-side bound of *kv_len the launch geometry was derived from
    int window_blocks;  // block sliding window in blocks of 128 keys (0 = none): key blocks below
                        // ceil(P / 128) - window_blocks are not visited (src/flash_attn/src/flash_blockmask.h:32,43-46)
    float scale_log2;
    f16* out;
    // Split partials in the accumulator's own layout, so that both the split kernel's stores and the
    // combine kernel's loads are whole 1 KB wave transactions:
    //   o_part  [Hkv][num_splits][rows_pad / 32 row blocks][16 quads][64 lanes] x 4 halves (normalised O)
    //           quad q = db * 4 + rq of lane (qcol, hf) holds O[row = block*32 + qcol][d = db*32 + rq*8 + hf*4 + 0..3]
    //   ml_part [Hkv][num_splits][rows_pad] x float2 (max * scale_log2, sum)
    float* o_part;
    float* ml_part;
    // Merge inside the split launch (null: the separate combine kernel does it): one word per (KV head, M-tile)
    // unit, arrivals in its low 16 bits, a generation count above them.  Between launches arrivals is 0; the last
    // workgroup of a unit to arrive turns the full count into the next generation.
    uint32_t* merge_ctr;
    uint32_t merge_wait_ticks;  // longest wait for the other workgroups of a unit, in ticks of the 100 MHz wall clock
};

constexpr int kMergeUnitWords = 64;  // a unit's word sits in a 256-byte line of its own: every poll and every arrival is
                                     // a memory transaction, and those on one line queue behind each other

// Loads and stores that other XCDs' workgroups of the same launch see: device-scope accesses go past the
// (per-XCD, mutually incoherent) L2.
__device__ inline uint64_t load_dev64(const void* ptr) {
    return __hip_atomic_load(reinterpret_cast<const uint64_t*>(ptr), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ inline void store_dev64(void* ptr, uint64_t v) {
    __hip_atomic_store(reinterpret_cast<uint64_t*>(ptr), v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
template <typename To, typename From>
__device__ inline To bits_as(const From& v) {
    static_assert(sizeof(To) == sizeof(From), "bits_as: size mismatch");
    return __builtin_bit_cast(To, v);
}

// Merge of the split partials of one 32-row block and one quad of output dims (one wave; lane = accumulator lane):
// M = max_s m_s, L = sum_s l_s 2^(m_s - M), O = sum_s l_s 2^(m_s - M) (O_s / l_s) / L -- the log-sum-exp merge of
// src/flash_attn/src/flash_fwd_kernel.h:2392-2472 in base-2 form.  The statistics and the O partials of up to 16
// splits are all requested before any is used, so a block pays one memory round trip, not one per split.
// DEV: the partials were written by other workgroups of this launch (device-scope loads).
constexpr int kCombineBatch = 16;
template <bool DEV, typename E>
__device__ inline void combine_block(const AttnParams& p, int g, int rb, int quad, int lane) {
    typedef typename Elem<E>::x4 X4;
    const int nrb = p.rows_pad / kRowsPerWave;  // 32-row blocks per kv head
    const int qcol = lane & 31, hf = lane >> 5;
    const int R = rb * kRowsPerWave + qcol;
    if (R >= p.group * p.T) return;
    const int node = p.group_shift >= 0 ? R >> p.group_shift : R / p.group;
    const int head = g * p.group + (p.group_shift >= 0 ? R & (p.group - 1) : R % p.group);
    const int d0 = (quad >> 2) * 32 + (quad & 3) * 8 + hf * 4;
    const float2* ml = reinterpret_cast<const float2*>(p.ml_part) + (size_t)g * p.num_splits * p.rows_pad + R;
    const X4* op = reinterpret_cast<const X4*>(p.o_part) +
                      (((size_t)g * p.num_splits) * nrb + rb) * 16 * 64 + quad * 64 + lane;
    const size_t ml_stride = (size_t)p.rows_pad;
    const size_t o_stride = (size_t)nrb * 16 * 64;

    float M = -INFINITY, L = 0.f;
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    for (int s0 = 0; s0 < p.num_splits; s0 += kCombineBatch) {
        float2 v[kCombineBatch];
        X4 o[kCombineBatch];
#pragma unroll
        for (int u = 0; u < kCombineBatch; ++u) {
            const int s = min(s0 + u, p.num_splits - 1);  // clamp: repeats are ignored below
            if (DEV) {
                const uint64_t mlw = load_dev64(&ml[s * ml_stride]);
                v[u] = make_float2(__uint_as_float((uint32_t)mlw), __uint_as_float((uint32_t)(mlw >> 32)));
                o[u] = bits_as<X4>(load_dev64(&op[s * o_stride]));
            } else {
                v[u] = ml[s * ml_stride];
                o[u] = op[s * o_stride];
            }
        }
        float Mb = M;
#pragma unroll
        for (int u = 0; u < kCombineBatch; ++u)
            if (s0 + u < p.num_splits && v[u].y > 0.f) Mb = fmaxf(Mb, v[u].x);
        if (Mb == -INFINITY) continue;  // nothing but empty splits so far
        const float resc = __builtin_amdgcn_exp2f(M - Mb);  // 0 when M was -inf
        L *= resc;
#pragma unroll
        for (int e = 0; e < 4; ++e) acc[e] *= resc;
        M = Mb;
#pragma unroll
        for (int u = 0; u < kCombineBatch; ++u) {
            // an empty split (l == 0) has no meaningful O partial: select it away, never scale it
            if (!(s0 + u < p.num_splits && v[u].y > 0.f)) continue;
            const float w = __builtin_amdgcn_exp2f(v[u].x - M) * v[u].y;  // partials are stored normalised
            L += w;
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[e] += w * (float)o[u][e];
        }
    }
    const float inv = (L == 0.f || L != L) ? 1.f : 1.f / L;
    X4 o;
#pragma unroll
    for (int e = 0; e < 4; ++e) o[e] = (E)(acc[e] * inv);
    *reinterpret_cast<X4*>(p.out + ((size_t)node * p.Hq + head) * kHeadDim + d0) = o;
}

// The same merge for more splits than a launch merges itself (more than kMergeMaxSplits: plain decode and small trees at long
// contexts), where combine_block's one batch after the other would be up to eight memory round trips: every batch of 16 is
// summed relative to its own maximum by a wave of its own, and one wave folds the batch sums in batch order.  (Another
// order of additions than combine_block's running sum: the two agree to rounding, not to the bit -- no launch has both.)
struct CombineSum {
    float M, L;
    f32x4 acc;
};
template <typename E>
struct CombineWhere {
    const float2* ml;
    const typename Elem<E>::x4* op;
    size_t ml_stride, o_stride;
    int node, head, d0;
    bool valid;
};
template <typename E>
__device__ inline CombineWhere<E> combine_where(const AttnParams& p, int g, int rb, int quad, int lane) {
    typedef typename Elem<E>::x4 X4;
    CombineWhere<E> w;
    const int nrb = p.rows_pad / kRowsPerWave;  // 32-row blocks per kv head
    const int qcol = lane & 31, hf = lane >> 5;
    const int R = rb * kRowsPerWave + qcol;
    w.valid = R < p.group * p.T;
    w.node = p.group_shift >= 0 ? R >> p.group_shift : R / p.group;
    w.head = g * p.group + (p.group_shift >= 0 ? R & (p.group - 1) : R % p.group);
    w.d0 = (quad >> 2) * 32 + (quad & 3) * 8 + hf * 4;
    w.ml = reinterpret_cast<const float2*>(p.ml_part) + (size_t)g * p.num_splits * p.rows_pad + R;
    w.op = reinterpret_cast<const X4*>(p.o_part) + (((size_t)g * p.num_splits) * nrb + rb) * 16 * 64 + quad * 64 + lane;
    w.ml_stride = (size_t)p.rows_pad;
    w.o_stride = (size_t)nrb * 16 * 64;
    return w;
}
// the sum over splits [s0, s0 + 16) relative to their own maximum; M = -inf, L = 0 when all of them are empty
template <bool DEV, typename E>
__device__ inline CombineSum combine_batch(const CombineWhere<E>& w, int s0, int num_splits) {
    typedef typename Elem<E>::x4 X4;
    float2 v[kCombineBatch];
    X4 o[kCombineBatch];
#pragma unroll
    for (int u = 0; u < kCombineBatch; ++u) {
        const int s = min(s0 + u, num_splits - 1);  // clamp: repeats are ignored below
        if (DEV) {
            const uint64_t mlw = load_dev64(&w.ml[s * w.ml_stride]);
            v[u] = make_float2(__uint_as_float((uint32_t)mlw), __uint_as_float((uint32_t)(mlw >> 32)));
            o[u] = bits_as<X4>(load_dev64(&w.op[s * w.o_stride]));
        } else {
            v[u] = w.ml[s * w.ml_stride];
            o[u] = w.op[s * w.o_stride];
        }
    }
    CombineSum r;
    r.M = -INFINITY;
    r.L = 0.f;
    r.acc = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int u = 0; u < kCombineBatch; ++u)
        if (s0 + u < num_splits && v[u].y > 0.f) r.M = fmaxf(r.M, v[u].x);
    if (r.M == -INFINITY) return r;
#pragma unroll
    for (int u = 0; u < kCombineBatch; ++u) {
        // an empty split (l == 0) has no meaningful O partial: select it away, never scale it
        if (!(s0 + u < num_splits && v[u].y > 0.f)) continue;
        const float wt = __builtin_amdgcn_exp2f(v[u].x - r.M) * v[u].y;  // partials are stored normalised
        r.L += wt;
#pragma unroll
        for (int e = 0; e < 4; ++e) r.acc[e] += wt * (float)o[u][e];
    }
    return r;
}
// folds a batch sum into the running result (the first batch into an empty one exactly: scale 0 and scale 1)
__device__ inline void combine_fold(CombineSum& t, const CombineSum& b) {
    if (b.M == -INFINITY) return;
    const float Mn = fmaxf(t.M, b.M);
    const float ra = __builtin_amdgcn_exp2f(t.M - Mn);  // 0 while the running result is empty
    const float rb = __builtin_amdgcn_exp2f(b.M - Mn);
    t.L = __builtin_fmaf(t.L, ra, b.L * rb);
#pragma unroll
    for (int e = 0; e < 4; ++e) t.acc[e] = __builtin_fmaf(t.acc[e], ra, b.acc[e] * rb);
    t.M = Mn;
}
template <typename E>
__device__ inline void combine_store(const AttnParams& p, const CombineWhere<E>& w, const CombineSum& t) {
    typedef typename Elem<E>::x4 X4;
    const float inv = (t.L == 0.f || t.L != t.L) ? 1.f : 1.f / t.L;
    X4 o;
#pragma unroll
    for (int e = 0; e < 4; ++e) o[e] = (E)(t.acc[e] * inv);
    *reinterpret_cast<X4*>(p.out + ((size_t)w.node * p.Hq + w.head) * kHeadDim + w.d0) = o;
}

// One rotary pair: (a, b) -> (a cos - b sin, a sin + b cos), every product and sum rounded on its own
// (no fused multiply-add), so the result does not depend on how a compiler contracts the expression.
template <typename E>
__device__ inline void rotate_pair(E& a, E& b, float2 cs) {
#pragma clang fp contract(off)
    const float fa = (float)a, fb = (float)b;
    const float ac = fa * cs.x, bs = fb * cs.y, as = fa * cs.y, bc = fb * cs.x;
    a = (E)(ac - bs);
    b = (E)(as + bc);
}

template <typename E>
__device__ inline typename Elem<E>::x8 zero8() {
    typename Elem<E>::x8 z;
#pragma unroll
    for (int i = 0; i < 8; ++i) z[i] = (E)0.f;
    return z;
}

// Swizzled LDS byte offsets inside one stage.  K: row = key (16 pieces of 16 B), piece index is
// XORed with key % 16.  V^T: row = dim (8 pieces), XORed with (dim / 2) % 8 -- even and odd rows
// already sit in different bank halves.  Both make the 16-byte MFMA operand reads conflict-free.
__device__ inline int k_lds_off(int key, int piece) { return key * 256 + ((piece ^ (key & 15)) << 4); }
__device__ inline int v_lds_off(int d, int piece) { return kKTileBytes + d * 128 + ((piece ^ ((d >> 1) & 7)) << 4); }

// One direct-to-LDS load: every lane fetches 16 bytes from its own global address and the wave's
// 1 KB lands at `lds_dst` (wave-uniform) in lane order.  Written as inline assembly on purpose: the
// completion of these loads is tracked by hand (s_waitcnt vmcnt before the workgroup barrier that
// publishes a stage), which lets the next tiles stay in flight while the current ones are consumed;
// with the compiler builtin every LDS read would first wait for all of them.
__device__ inline void load_to_lds16(const void* base, uint32_t byte_off, const char* lds_dst) {
    const uint32_t lds_addr = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(lds_ptr_t)lds_dst);
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" : : "v"(byte_off), "s"(base), "s"(lds_addr) : "memory", "m0");
}

// Four bytes per lane (256 bytes per wave instruction), full per-lane address.
__device__ inline void load_to_lds4_v(const void* gptr, const char* lds_dst) {
    const uint32_t lds_addr = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(lds_ptr_t)lds_dst);
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dword %0, off" : : "v"(gptr), "s"(lds_addr) : "memory", "m0");
}

// Same, with a full per-lane address (used where lanes of one instruction read from different buffers).
__device__ inline void load_to_lds16_v(const void* gptr, const char* lds_dst) {
    const uint32_t lds_addr = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(lds_ptr_t)lds_dst);
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(gptr), "s"(lds_addr) : "memory", "m0");
}

// Scalar loads of wave-uniform int32 values, issued and awaited in place: an entry of the page table when a tile is
// requested (consecutive entries share a cache line, so after the first one of a page run these are scalar-cache
// hits), and the KV length together with the first page id at the start of the kernel, where a vector load would
// queue behind the Q rows.  Nothing else of this wave's scalar or LDS traffic is outstanding at those points.
__device__ inline int scalar_load(const int32_t* ptr) {
    int v;
    asm volatile("s_load_dword %0, %1, 0x0\n\ts_waitcnt lgkmcnt(0)" : "=s"(v) : "s"(ptr) : "memory");
    return v;
}
__device__ inline void scalar_load2(const int32_t* pa, const int32_t* pb, int& a, int& b) {
    asm volatile("s_load_dword %0, %2, 0x0\n\ts_load_dword %1, %3, 0x0\n\ts_waitcnt lgkmcnt(0)" : "=&s"(a), "=&s"(b) : "s"(pa), "s"(pb) : "memory");
}
__device__ inline void scalar_load3(const int32_t* pa, const int32_t* pb, const int32_t* pc, int& a, int& b, int& c) {
    asm volatile("s_load_dword %0, %3, 0x0\n\ts_load_dword %1, %4, 0x0\n\ts_load_dword %2, %5, 0x0\n\ts_waitcnt lgkmcnt(0)"
                 : "=&s"(a), "=&s"(b), "=&s"(c) : "s"(pa), "s"(pb), "s"(pc) : "memory");
}

// Per-thread byte offsets of its pieces inside a K tile and a V^T tile of a page (second piece of each:
// + 32 keys = 8192 bytes for K, + 64 dims = 64 * 512 bytes for V^T; the swizzle terms do not change).
__device__ inline uint32_t k_piece_off(int wave, int lane) {
    const int key = wave * 4 + (lane >> 4);
    const int piece = (lane & 15) ^ (key & 15);
    return (uint32_t)(key * kHeadDim + piece * 8) * 2u;
}
__device__ inline uint32_t v_piece_off(int wave, int lane) {
    const int d = wave * 8 + (lane >> 3);
    const int piece = (lane & 7) ^ ((d >> 1) & 7);
    return (uint32_t)(d * kPage + piece * 8) * 2u;
}

// Issues this thread's four 16-byte direct-to-LDS loads of one tile (2 for K, 2 for V^T).  Each
// wave-level instruction fills 1 KB of LDS in lane order; the swizzle is applied on the global side.
// Everything but the two per-thread offsets is wave-uniform, so the address arithmetic is scalar.
__device__ inline void issue_tile(const AttnParams& p, int g, int tile, int page, char* stage, int wave, uint32_t koff, uint32_t voff) {
    const int slot0 = (tile * kTileN) % kPage;
    const char* kbase = reinterpret_cast<const char*>(p.k_pool + (((size_t)page * p.Hkv + g) * kPage + slot0) * kHeadDim);
    const char* vbase = reinterpret_cast<const char*>(p.v_pool + ((size_t)page * p.Hkv + g) * kHeadDim * kPage + slot0);
    load_to_lds16(kbase, koff, stage + wave * 1024);
    load_to_lds16(vbase, voff, stage + kKTileBytes + wave * 1024);
    load_to_lds16(kbase + 32 * kHeadDim * 2, koff, stage + (wave + kWaves) * 1024);
    load_to_lds16(vbase + 64 * kPage * 2, voff, stage + kKTileBytes + (wave + kWaves) * 1024);
}

// The same for a tile that reaches the rows being appended: keys at positions [P, S) take their K
// pieces straight from k_new (same 16-byte pieces, so the fused append costs K nothing); V^T comes
// from the pool as usual and is patched in LDS afterwards.
__device__ inline void issue_tile_append(const AttnParams& p, int g, int tile, int page, char* stage, int wave, int lane, uint32_t koff,
                                         uint32_t voff, int P, int S) {
    const int slot0 = (tile * kTileN) % kPage;
    const char* kbase = reinterpret_cast<const char*>(p.k_pool + (((size_t)page * p.Hkv + g) * kPage + slot0) * kHeadDim);
    const char* vbase = reinterpret_cast<const char*>(p.v_pool + ((size_t)page * p.Hkv + g) * kHeadDim * kPage + slot0);
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        const int key = h * 32 + wave * 4 + (lane >> 4);
        const int c = tile * kTileN + key;
        const int piece = (lane & 15) ^ (key & 15);
        const char* src = kbase + h * (32 * kHeadDim * 2) + koff;
        if (c >= P && c < S) src = reinterpret_cast<const char*>(p.k_new + ((size_t)(c - P) * p.Hkv + g) * kHeadDim + piece * 8);
        load_to_lds16_v(src, stage + (wave + kWaves * h) * 1024);
        load_to_lds16(vbase + h * (64 * kPage * 2), voff, stage + kKTileBytes + (wave + kWaves * h) * 1024);
    }
}

// ROPE: the instantiation that rotates q and the appended K rows (p.rope is set); the plain one carries
// none of that code, so its registers and schedule are those of a kernel without the feature.
// E: the element type.  The kernels proper are thin wrappers below (`tree_attn_split_kernel<G, ROPE>` for fp16 keeps the name
// it has in every profile, `tree_attn_split_bf16_kernel<G, ROPE>` for bf16).
template <int G, bool ROPE, typename E>
__device__ __forceinline__ void tree_attn_split_body(const AttnParams& p) {
    typedef typename Elem<E>::x8 X8;
    typedef typename Elem<E>::x4 X4;
    typedef typename Elem<E>::x2 X2;
    constexpr int kRowWaves = kWaves / G;
    constexpr int kRowsPerWg = kRowWaves * kRowsPerWave;
    constexpr int kDepth = kStages / G - 1;  // iterations in flight behind the one being consumed
    __shared__ __attribute__((aligned(1024))) char ring[kStages * kStageBytes];
    __shared__ __attribute__((aligned(1024))) char vstage[kVStageRows * kHeadDim * 2];  // first appended V rows, row-major
    __shared__ uint64_t s_mask[kMaxTree * 2];                                            // the tree mask as handed in
    __shared__ int s_append_page[3];  // pages of the (at most three: T <= 128) tiles that hold appended rows, as their requests found them

    // XCD-aware work mapping: the grid is (splits x KV heads, padded to a multiple of the XCD count) x M-tiles.
    // Workgroups are numbered x first and consecutive numbers go to consecutive XCDs, so x % 8 picks the XCD:
    // all M-tiles of one (split, kv head) pair share an XCD and the K/V pages they stream meet in its L2.
    // All launch arguments are fetched in one go, up front: left alone, the compiler fetches them in three batches as
    // the code first needs them, and each batch is a memory round trip of its own in front of the first K/V request.
    asm volatile("" ::"s"(p.q), "s"(p.k_pool), "s"(p.v_pool), "s"(p.block_table), "s"(p.kv_len), "s"(p.k_new), "s"(p.v_new), "s"(p.rope),
                 "s"(p.mask), "s"(p.mask_words), "s"(p.mask_k_range), "s"(p.T), "s"(p.Hq), "s"(p.Hkv), "s"(p.group), "s"(p.group_shift),
                 "s"(p.hkv_shift), "s"(p.num_splits), "s"(p.num_mtiles), "s"(p.ntiles_max), "s"(p.table_pages), "s"(p.window_blocks),
                 "s"(p.max_kv_len));
    CPMCU_CLOCK_VAR(tl_start);
    CPMCU_CLOCK_VAR(tl_loop);
    CPMCU_CLOCK_VAR(tl_loop_end);
    CPMCU_CLOCK_VAR(tl_groups);
    CPMCU_CLOCK_VAR(tl_stored);
    CPMCU_CLOCK_VAR(tl_acked);
    CPMCU_CLOCK_VAR(tl_go);
    CPMCU_CLOCK_VAR(tl_it1);
    CPMCU_CLOCK_VAR(tl_it2);
    CPMCU_CLOCK_VAR(tl_fix0);
    CPMCU_CLOCK_VAR(tl_fix1);
    CPMCU_CLOCK(tl_start);
    const int sh = blockIdx.x;
    const int mt = blockIdx.y;
    if (sh >= p.num_splits * p.Hkv) return;
    const int g = p.hkv_shift >= 0 ? sh & (p.Hkv - 1) : sh % p.Hkv;
    const int split = p.hkv_shift >= 0 ? sh >> p.hkv_shift : sh / p.Hkv;

    const int tid = threadIdx.x;
    const int wave = tid >> 6;
    const int lane = tid & 63;
    uint32_t* const unit_ctr = p.merge_ctr ? p.merge_ctr + kMergeUnitWords * (g * p.num_mtiles + mt) : nullptr;  // merge inside the launch
    const int grp = wave / kRowWaves;  // KV group: takes tiles grp, grp + G, ...
    const int rw = wave % kRowWaves;
    const int qcol = lane & 31;
    const int hf = lane >> 5;

    const int R = mt * kRowsPerWg + rw * kRowsPerWave + qcol;  // packed row
    const bool row_ok = R < p.group * p.T;
    // A wave whose 32 rows all lie past the last packed row (the tail of the last M-tile: two of its eight waves for a
    // 60-node tree) has nothing to compute: it still requests its share of every tile and meets every barrier, but
    // skips the tile arithmetic -- 6 % of the launch's matrix and vector work at that tree size.
    const bool wave_has_rows = __builtin_amdgcn_readfirstlane(mt * kRowsPerWg + rw * kRowsPerWave) < p.group * p.T;
    const int node = !row_ok ? 0 : p.group_shift >= 0 ? R >> p.group_shift : R / p.group;
    const int head = g * p.group + (!row_ok ? 0 : p.group_shift >= 0 ? R & (p.group - 1) : R % p.group);

    // Loads that do not depend on the KV length go first.
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);
    // The tree mask (src/flash_attn/src/mask.h:185-198; at most 128 rows of two words) goes to LDS whole, one request
    // per wave, and is awaited together with the Q rows below (requests return in order): a load into registers here
    // would have the compiler wait for everything in flight at the mask's first use.
    if (p.mask) {
        const int ndw = p.T * p.mask_words * 2;
        load_to_lds4_v(reinterpret_cast<const uint32_t*>(p.mask) + min(wave_u * 64 + lane, ndw - 1), reinterpret_cast<const char*>(s_mask) + wave_u * 256);
    }
    // The workgroup's Q rows go to LDS first, as whole 256-byte rows (four rows per wave instruction), into the
    // ring stages the first tile requests leave free, and are read from there into the B-operand registers:
    // fetched straight into that layout -- every lane 16 bytes of a row of its own -- a wave instruction touches
    // 32 cache lines for 1 KB and the eight of them hold the CU's address path for 1.5 us ahead of the first K/V
    // tile.  Both KV groups read the same copy.
    constexpr int kQStages = kRowsPerWg * kHeadDim * 2 / kStageBytes;  // ring stages the Q rows occupy
    char* const qstage = ring + (kStages - kQStages) * kStageBytes;
    auto issue_q = [&]()     {
        const int last_row = p.group * p.T - 1;
#pragma unroll
        for (int x = 0; x < kRowsPerWg / (4 * kWaves); ++x) {
            const int inst = x * kWaves + wave_u;  // 1 KB of the staging area: rows 4 * inst .. + 3
            const int r = inst * 4 + (lane >> 4);
            const int Rr = min(mt * kRowsPerWg + r, last_row);  // rows past the end re-read the last one (zeroed below)
            const int nr = p.group_shift >= 0 ? Rr >> p.group_shift : Rr / p.group;
            const int hr = g * p.group + (p.group_shift >= 0 ? Rr & (p.group - 1) : Rr % p.group);
            const int piece = (lane & 15) ^ (r & 15);  // the K tile's swizzle: the reads below are conflict-free
            load_to_lds16_v(p.q + ((size_t)nr * p.Hq + hr) * kHeadDim + piece * 8, qstage + inst * 1024);
        }
    };

    // The split ranges partition the tiles of the stream as the device-side length gives it, so that every split gets its
    // share of what is really there (a padded host-side bound would leave the last splits short and the others long).
    // The page id of the split's first tile is still fetched together with the length, not behind it: the exact first
    // tile can only lie at or below the one the host-side bound gives, almost always on the same page or the one before,
    // so both table entries are requested with the length; a first tile further away (a bound far above the length)
    // costs one more scalar load.
    // With the fused append the last split also patches the appended rows into its tiles, which costs
    // about as much as an iteration: the partition counts two tiles' worth of extra work at the end
    // of the stream (three when the appended K rows are also rotated there), so that split gets fewer real tiles.
    // A block sliding window moves the start of the stream to its first visible tile, which depends on
    // the device-side length: such calls (the drafter's own layer, a few tiles in all) pay the extra
    // round trip in front of the page ids and keep the partition of the window's bound.
    const int extra_tiles = p.k_new != nullptr && p.num_splits > 1 ? (ROPE ? 3 : 2) : 0;
    // (32-bit arithmetic: at most 128 splits times at most 2^24 tiles; a 64-bit division is a long scalar routine)
    auto range_begin = [&](int sp, int tiles) { return min((int)(((uint32_t)sp * (uint32_t)(tiles + extra_tiles)) / (uint32_t)p.num_splits), tiles); };
    int S, first_page;
    int tile_lo = 0;
    int r0, r1;
    auto clamp_length = [&]() {
        const int lo = max(p.T, p.mask_k_range);
        if (S > p.max_kv_len || S < lo) {
            if (sh == 0 && mt == 0 && tid == 0) g_attn_report.bad_length = S == 0 ? -1 : S;
            S = min(max(S, lo), p.max_kv_len);
        }
    };
    if (p.window_blocks > 0) {  // the window's first tile depends on the length: one more round trip for the page id
        S = scalar_load(p.kv_len);
        clamp_length();
        r0 = range_begin(split, p.ntiles_max);
        r1 = range_begin(split + 1, p.ntiles_max);
        tile_lo = max((S - p.T + 127) / 128 - p.window_blocks, 0) * (128 / kTileN);
        first_page = scalar_load(p.block_table + min(((tile_lo + r0) * kTileN) / kPage, p.table_pages - 1));
    } else {
        const int pg_b = min((range_begin(split, p.ntiles_max) * kTileN) / kPage, p.table_pages - 1);
        int page_b, page_before;
        scalar_load3(p.kv_len, p.block_table + pg_b, p.block_table + max(pg_b - 1, 0), S, page_b, page_before);
        clamp_length();
        const int ntiles_now = (S + kTileN - 1) / kTileN;
        r0 = range_begin(split, ntiles_now);
        r1 = range_begin(split + 1, ntiles_now);
        const int pg = min((r0 * kTileN) / kPage, p.table_pages - 1);
        first_page = pg == pg_b ? page_b : pg == pg_b - 1 ? page_before : scalar_load(p.block_table + pg);
    }
    const int t0 = tile_lo + r0;
    const int t1_max = tile_lo + r1;
    const int pg0 = min((t0 * kTileN) / kPage, p.table_pages - 1);
    // page of a tile: a scalar load of its table entry (the first one is already here)
    // (a window's last tile slot can lie past the host bound; it is never consumed, and the table is not read there)
    auto page_of_tile = [&](int tile) {
        const int pg = min((tile * kTileN) / kPage, p.table_pages - 1);
        return pg == pg0 ? first_page : scalar_load(p.block_table + pg);
    };
    const int P = S - p.T;              // the T query tokens are the last T keys
    const int Pm = S - p.mask_k_range;  // first key column governed by the mask bits (mask.h: mask_k_begin)
    const int ntiles = (S + kTileN - 1) / kTileN;
    const int t1 = min(t1_max, ntiles);
    const int n = max(t1 - t0, 0);
    const int niter = (n + G - 1) / G;  // one iteration consumes G tiles, one per KV group

    const uint32_t koff = k_piece_off(wave, lane), voff = v_piece_off(wave, lane);
    auto issue_tile_i = [&](int i) {  // the i-th tile of this workgroup's range, into its ring stage
        const int tile = t0 + i;
        const int page = page_of_tile(tile);
        if (p.k_new != nullptr && (tile + 1) * kTileN > P) {
            // (the page is kept for the patch of the landed tile: a table load there would sit in front of its LDS reads)
            if (tid == 0) s_append_page[min(max(tile - P / kTileN, 0), 2)] = page;
            issue_tile_append(p, g, tile, page, ring + (i % kStages) * kStageBytes, wave_u, lane, koff, voff, P, S);
        } else
            issue_tile(p, g, tile, page, ring + (i % kStages) * kStageBytes, wave_u, koff, voff);
    };
    auto issue_iter = [&](int it) {
#pragma unroll
        for (int e = 0; e < G; ++e)
            if (it * G + e < n) issue_tile_i(it * G + e);
    };

    f32x16 oacc[4];
#pragma unroll
    for (int db = 0; db < 4; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) oacc[db][r] = 0.f;
    // Online softmax state of this lane's query row.  m_ref is the exponent reference in log2 units
    // (score * scale * log2 e): probabilities are computed as 2^(s - m_ref).  It follows the running
    // row maximum lazily -- it is raised (and O, l rescaled) only when a tile's maximum exceeds it by
    // more than kLazyLog2, so the rescale of the 64 accumulator registers is rare; meanwhile
    // probabilities may reach 2^kLazyLog2, far inside fp16 and fp32 range.  O / l does not depend
    // on the reference.
    float m_ref = -INFINITY;
    float l_run = 0.f;        // this lane's share of the row sum

    // A workgroup whose range reaches the tree region transposes the appended V rows into its tiles.
    // The first kVStageRows of them are requested into LDS now -- the oldest loads, so the first wait
    // below covers them -- and the latency of reading v_new stays off the critical path.
    if (p.k_new != nullptr && (t0 + n) * kTileN > P) {
#pragma unroll
        for (int qq = 0; qq < 2; ++qq) {
            const int inst = wave_u + kWaves * qq;
            const int r = min(inst * 4 + (lane >> 4), p.T - 1);
            load_to_lds16_v(p.v_new + ((size_t)r * p.Hkv + g) * kHeadDim + (lane & 15) * 8, vstage + inst * 1024);
        }
    }
    // The first tiles are requested into the stages the Q rows do not occupy ...
    constexpr int kPrologueTiles = (kDepth + 1) * G;  // = kStages
    constexpr int kEarlyTiles = kStages - kQStages;
    const int n_early = min(n, kEarlyTiles);
    constexpr int kFirstTiles = G;  // the first iteration's tiles go ahead of the Q rows
#pragma unroll
    for (int i = 0; i < kFirstTiles; ++i)
        if (i < n) issue_tile_i(i);
    issue_q();
#pragma unroll
    for (int i = kFirstTiles; i < kEarlyTiles; ++i)
        if (i < n) issue_tile_i(i);
    // ... then the Q rows (and the mask words, older still) are awaited: everything requested after them may stay in flight
    // (4 loads per thread and tile; the two staged V requests, where issued, are waited for as well).
    switch (n_early - min(n, kFirstTiles)) {
        case 0: asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); break;
        case 1: asm volatile("s_waitcnt vmcnt(4)" ::: "memory"); break;
        case 2: asm volatile("s_waitcnt vmcnt(8)" ::: "memory"); break;
        default: asm volatile("s_waitcnt vmcnt(12)" ::: "memory"); break;
    }
    __syncthreads();
    uint64_t mw0 = ~0ull, mw1 = ~0ull;
    if (p.mask) {
        mw0 = s_mask[node * p.mask_words];
        mw1 = p.mask_words > 1 ? s_mask[node * p.mask_words + 1] : 0ull;
    }
    // Q as the B operand of S^T = K.Q^T: lane (qcol, hf) holds d = 16*ks + 8*hf + [0,8).
    X8 qreg[8];
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) {
        const X8 v = *reinterpret_cast<const X8*>(qstage + k_lds_off(rw * kRowsPerWave + qcol, 2 * ks + hf));
        qreg[ks] = row_ok ? v : zero8<E>();
    }
    __syncthreads();  // the stages are free for tiles
#pragma unroll
    for (int i = kEarlyTiles; i < kPrologueTiles; ++i)
        if (i < n) issue_tile_i(i);
    {
        // the causal bound j <= node folded into the mask row: the mask column of the query's own key is kept,
        // every column above it cleared
        const int own = p.mask_k_range - p.T + node;
        const uint64_t c0 = own >= 63 ? ~0ull : ((2ull << own) - 1ull);
        const uint64_t c1 = own >= 127 ? ~0ull : (own < 64 ? 0ull : ((2ull << (own - 64)) - 1ull));
        mw0 &= c0;
        mw1 &= c1;
    }

    // Fused rotary embedding of the query (rotary_embedding_kernel, src/model/rotary.cuh:11-22), placed behind
    // the first tile requests so that its table reads and arithmetic run under their latency: the pair
    // (d, d + 64) of a row sits in the same lane, registers ks and ks + 4, and rotates by the angle
    // of (node position, d); products in fp32, results rounded to fp16 as the in-place kernel leaves them.
    if (ROPE && row_ok) {
        const float2* cs = p.rope + (size_t)node * (kHeadDim / 2) + hf * 8;
#pragma unroll
        for (int ks = 0; ks < 4; ++ks)
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                E a = qreg[ks][j], b = qreg[ks + 4][j];
                rotate_pair(a, b, cs[ks * 16 + j]);
                qreg[ks][j] = a;
                qreg[ks + 4][j] = b;
            }
    }

    CPMCU_CLOCK(tl_loop);
    for (int it = 0; it < niter; ++it) {
        // Wait for this iteration's tiles.  The prologue issued iterations 0..kDepth and iteration
        // j >= 1 issues iteration j + kDepth right after its barrier, so the tiles issued so far are
        // those of iterations <= max(it - 1, 0) + kDepth; the ones beyond this iteration (4 loads per
        // thread and tile, returned in order) may stay in flight.
        // The first iteration's tiles were requested ahead of the Q rows, so the wait and the barriers of the prologue
        // have covered them: the two-group shape, whose launches are short, goes straight on (0.25 us of 15.6 per
        // layer at 4K); the 256-row shape keeps the uniform loop (without it 47.5 vs 46.2 us at 32K).
        if (G == 1 || it > 0) {
            const int issued = min(n, (max(it - 1, 0) + kDepth + 1) * G);
            const int needed = min(n, (it + 1) * G);
            switch (issued - needed) {
                case 0: asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); break;
                case 1: asm volatile("s_waitcnt vmcnt(4)" ::: "memory"); break;
                case 2: asm volatile("s_waitcnt vmcnt(8)" ::: "memory"); break;
                default: asm volatile("s_waitcnt vmcnt(12)" ::: "memory"); break;
            }
            __syncthreads();  // every thread's pieces have landed; the previous iteration's stages are free
        }
        if (it >= 1 && it + kDepth < niter) issue_iter(it + kDepth);

        const int i = it * G + grp;  // this group's tile of the iteration
        const int t = t0 + i;
        const int c0 = t * kTileN;
        char* stage = ring + (i % kStages) * kStageBytes;
        // Fix-ups of landed tiles, in LDS (uniform over the workgroup: only the pairs that reach the
        // tree region or the end of the stream pay for them):
        //  * fused KV append (copy_to_kvcache, src/model/attn.cuh:14-21,200): when the T new rows are
        //    handed in, they replace whatever the cache held at positions [P, S) -- every workgroup
        //    patches its own LDS copy, and the M-tile-0 workgroup of the split also writes the rows
        //    into the paged pools;
        //  * the tile that holds position S-1 may extend past it: stale page contents there must not
        //    reach the MFMA (0 * NaN = NaN), so the V^T columns of tokens >= S are zeroed.  K needs
        //    nothing: the scores of those keys are replaced (not scaled) by -inf below.
#ifdef CPMCU_TIMELINE
        if (it == 1) tl_it1 = wall_clock64();
#endif
        const int iter_end = (t0 + it * G) * kTileN + G * kTileN;
        const bool iter_needs_fix = iter_end > S || (p.k_new != nullptr && iter_end > P);
        if (iter_needs_fix) {
            for (int e = 0; e < G; ++e) {
                const int ie = it * G + e;
                const int ce = (t0 + ie) * kTileN;
                if (ie >= n) continue;
                char* st = ring + (ie % kStages) * kStageBytes;
                const bool append = p.k_new != nullptr && ce + kTileN > P;
                // a tile lies inside one page; the id was left in LDS when the tile was requested (a barrier ago at least)
                const int pg = !append ? 0 : __builtin_amdgcn_readfirstlane(s_append_page[min(max(t0 + ie - P / kTileN, 0), 2)]);
                if (ROPE && append) {
                    // Fused rotary embedding of the appended K rows (src/model/rotary.cuh:23-33): the tile holds
                    // them as fetched from k_new; one thread per (key, 16-byte piece of the lower half) rotates
                    // the piece with its partner 64 dims up, in LDS, and the M-tile-0 workgroup passes the
                    // rotated pieces on to the pool.
                    for (int x = tid; x < kTileN * 8; x += kThreads) {
                        const int key = x >> 3, piece = x & 7;
                        const int c = ce + key;
                        if (c >= P && c < S) {
                            X8* lo = reinterpret_cast<X8*>(st + k_lds_off(key, piece));
                            X8* hi = reinterpret_cast<X8*>(st + k_lds_off(key, piece + 8));
                            X8 a = *lo, b = *hi;
                            const float2* cs = p.rope + (size_t)(c - P) * (kHeadDim / 2) + piece * 8;
#pragma unroll
                            for (int j = 0; j < 8; ++j) {
                                E ra = a[j], rb = b[j];
                                rotate_pair(ra, rb, cs[j]);
                                a[j] = ra;
                                b[j] = rb;
                            }
                            *lo = a;
                            *hi = b;
                            if (mt == 0) {
                                f16* row = p.k_pool_w + (((size_t)pg * p.Hkv + g) * kPage + c % kPage) * kHeadDim;
                                *reinterpret_cast<X8*>(row + piece * 8) = a;
                                *reinterpret_cast<X8*>(row + (piece + 8) * 8) = b;
                            }
                        }
                    }
                } else if (append && mt == 0) {
                    // K is already in the tile (fetched from k_new): the M-tile-0 workgroup copies the new
                    // rows' 16-byte pieces on to the pool.
                    for (int x = tid; x < kTileN * 16; x += kThreads) {
                        const int key = x >> 4, piece = x & 15;
                        const int c = ce + key;
                        if (c >= P && c < S)
                            *reinterpret_cast<f16x8*>(p.k_pool_w + (((size_t)pg * p.Hkv + g) * kPage + c % kPage) * kHeadDim + piece * 8) =
                                *reinterpret_cast<const f16x8*>(st + k_lds_off(key, piece));
                    }
                }
                CPMCU_CLOCK(tl_it2);
                if (append || ce + kTileN > S) {
                    // V^T, one 16-byte piece (8 token slots of one dim) per thread, read-modify-write:
                    // slots of appended tokens take the value from the staged row-major copy (the
                    // transposition), slots at or beyond S become zero, the others keep the pool's value.
                    // Trees of more than kVStageRows nodes read the rows beyond the staging area from
                    // v_new; the choice is uniform, so the usual case issues no global load here.
                    auto patch_v = [&](auto all_staged_c) {
                        constexpr bool kAllStaged = decltype(all_staged_c)::value;
                        // A wave works on one group of 8 token slots at a time, so which of them are appended rows, which lie
                        // beyond the end and which staged row each takes its value from are scalar quantities: the per-slot
                        // index arithmetic and the case distinctions stay off the vector pipe.
                        static_assert(kThreads % kHeadDim == 0 && (kHeadDim * 8) % kThreads == 0, "whole waves per slot group");
                        const int d = tid & (kHeadDim - 1);
#pragma unroll
                        for (int pass = 0; pass < (kHeadDim * 8) / kThreads; ++pass) {
                            const int sg = __builtin_amdgcn_readfirstlane(tid / kHeadDim + pass * (kThreads / kHeadDim));
                            f16x8* pp = reinterpret_cast<f16x8*>(st + v_lds_off(d, sg));
                            f16x8 cur = *pp;
                            bool has_new = false;
                            // all eight staged values are read unconditionally (clamped index) and selected
                            // afterwards: conditional reads would each wait for their own LDS round trip
                            uint16_t nv[8];
#pragma unroll
                            for (int j = 0; j < 8; ++j) {
                                const int r = min(max(ce + v_slot16(sg * 8 + j) - P, 0), kAllStaged ? p.T - 1 : kVStageRows - 1);
                                nv[j] = reinterpret_cast<const uint16_t*>(vstage)[r * kHeadDim + d];
                            }
                            if constexpr (kAllStaged) {
                                // The eight slots of a group are two runs of four consecutive token positions (v_slot16
                                // swaps bits 2 and 3 of the slot number), so which of them take the staged value
                                // ([P, S)), keep the pool's (below P, or below S when nothing is appended) or become
                                // zero (from S on) are two bit ranges per run: a handful of scalar instructions and one
                                // and-or per 64 bits, where a comparison chain per slot cost more than the tile's MFMAs.
                                uint64_t w2[2] = {__builtin_bit_cast(uint4, cur).x | ((uint64_t)__builtin_bit_cast(uint4, cur).y << 32),
                                                  __builtin_bit_cast(uint4, cur).z | ((uint64_t)__builtin_bit_cast(uint4, cur).w << 32)};
#pragma unroll
                                for (int h = 0; h < 2; ++h) {
                                    const int c0 = ce + v_slot16(sg * 8 + 4 * h);
                                    const int end = min(max(S - c0, 0), 4);
                                    const int beg = append ? min(max(P - c0, 0), end) : end;
                                    const uint64_t below_end = end >= 4 ? ~0ull : (1ull << (16 * end)) - 1ull;
                                    const uint64_t below_beg = beg >= 4 ? ~0ull : (1ull << (16 * beg)) - 1ull;
                                    const uint64_t staged = (uint64_t)nv[4 * h] | ((uint64_t)nv[4 * h + 1] << 16) | ((uint64_t)nv[4 * h + 2] << 32) |
                                                            ((uint64_t)nv[4 * h + 3] << 48);
                                    w2[h] = (staged & below_end & ~below_beg) | (w2[h] & below_beg);
                                    has_new = has_new || end > beg;
                                }
                                cur = __builtin_bit_cast(f16x8, make_uint4((uint32_t)w2[0], (uint32_t)(w2[0] >> 32), (uint32_t)w2[1], (uint32_t)(w2[1] >> 32)));
                            } else {
#pragma unroll
                                for (int j = 0; j < 8; ++j) {
                                    const int c = ce + v_slot16(sg * 8 + j);
                                    if (append && c >= P && c < S) {
                                        if (c - P < kVStageRows) cur[j] = __builtin_bit_cast(f16, nv[j]);
                                        else cur[j] = p.v_new[((size_t)(c - P) * p.Hkv + g) * kHeadDim + d];
                                        has_new = true;
                                    } else if (c >= S) {
                                        cur[j] = (f16)0.f;
                                    }
                                }
                            }
                            *pp = cur;
                            if (has_new && mt == 0)  // the same 8 slots are 16 contiguous bytes of the pool's page row
                                *reinterpret_cast<f16x8*>(p.v_pool_w + (((size_t)pg * p.Hkv + g) * kHeadDim + d) * kPage + ce % kPage + sg * 8) = cur;
                        }
                    };
                    if (p.T <= kVStageRows) patch_v(std::true_type{});
                    else patch_v(std::false_type{});
                }
            }
            CPMCU_CLOCK(tl_fix0);
            __syncthreads();
            CPMCU_CLOCK(tl_fix1);
        }
        if (i < n && wave_has_rows) {
            // ---- S^T = K.Q^T : two 32-key blocks.  All 16 operand reads are issued before the first
            // MFMA: LDS returns in order, so MFMA i only waits for read i. ----
            f32x16 sacc[2];
            {
                X8 kf[16];
#pragma unroll
                for (int ks = 0; ks < 8; ++ks)
#pragma unroll
                    for (int kb = 0; kb < 2; ++kb)
                        kf[ks * 2 + kb] = *reinterpret_cast<const X8*>(stage + k_lds_off(kb * 32 + qcol, 2 * ks + hf));
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                    for (int r = 0; r < 16; ++r) sacc[kb][r] = 0.f;
#pragma unroll
                for (int ks = 0; ks < 8; ++ks)
#pragma unroll
                    for (int kb = 0; kb < 2; ++kb)  // two independent accumulation chains, interleaved
                        sacc[kb] = Elem<E>::mfma_32x32x16(kf[ks * 2 + kb], qreg[ks], sacc[kb]);
                __builtin_amdgcn_sched_barrier(0);
            }
            // The V^T operands of this tile are requested now, so that they arrive under the softmax
            // arithmetic and the probability MFMAs start without waiting for LDS.
            X8 vf[16];
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int db = 0; db < 4; ++db)
                    vf[j * 4 + db] = *reinterpret_cast<const X8*>(stage + v_lds_off(db * 32 + qcol, 2 * j + hf));
            __builtin_amdgcn_sched_barrier(0);
            // sacc[kb][r] is the score of key  c0 + kb*32 + 8*(r/4) + 4*hf + r%4  for query qcol.
            if (c0 + kTileN > Pm) {  // tile touches masked columns or the end of the stream
                // 64-bit visibility word of this tile for the lane's query: bit x <-> key c0 + x.  Prefix
                // keys are visible; tree key P + j is visible iff bit j of the node's mask row is set
                // (the causal bound already cleared every bit above the node, hence at or beyond T).
                const int sh = Pm - c0;  // < 64 here; negative once the tile starts inside the masked range
                uint64_t tmask;
                if (sh >= 0) {
                    tmask = (mw0 << sh) | (sh > 0 ? ((1ull << sh) - 1ull) : 0ull);
                } else {
                    const int tt = -sh;
                    tmask = tt < 64 ? ((mw0 >> tt) | (mw1 << (64 - tt))) : (tt < 128 ? (mw1 >> (tt - 64)) : 0ull);
                }
                const uint64_t tm = tmask >> (4 * hf);
#pragma unroll
                for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const bool vis = (tm >> (kb * 32 + 8 * (r >> 2) + (r & 3))) & 1ull;
                        sacc[kb][r] = vis ? sacc[kb][r] : -INFINITY;
                    }
            }
            // ---- online softmax (one query column per lane) ----
            float tmax = sacc[0][0];
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int r = 0; r < 16; ++r) tmax = fmaxf(tmax, sacc[kb][r]);
            {   // The row's other half of the keys lives 32 lanes away: one cross-half register swap instead of
            // an LDS shuffle.  Written as assembly because the compiler builtin of this instruction hands
            // back its first result twice.  The two wait states cover the vector write of tmax just before.
            float mine = tmax, other = tmax;
            asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(mine), "+v"(other));
            tmax = fmaxf(mine, other) * p.scale_log2;  // scale > 0
        }
        if (__any(tmax > m_ref + kLazyLog2)) {  // some row's maximum moved far: re-reference all rows
                const float m_new = fmaxf(m_ref, tmax);
                const float alpha = (m_new == -INFINITY) ? 1.f : __builtin_amdgcn_exp2f(m_ref - m_new);
                m_ref = m_new;
                l_run *= alpha;
#pragma unroll
                for (int db = 0; db < 4; ++db)
#pragma unroll
                    for (int r = 0; r < 16; ++r) oacc[db][r] *= alpha;
            }
            const float m_scaled = (m_ref == -INFINITY) ? 0.f : m_ref;
            float psum = 0.f;
            X8 pb[4];  // P^T as B operand: k-step j holds keys 16*j + {4hf..4hf+3, 8+4hf..8+4hf+3}
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const float pv = __builtin_amdgcn_exp2f(sacc[kb][r] * p.scale_log2 - m_scaled);
                    pb[kb * 2 + (r >> 3)][r & 7] = (E)pv;  // P is rounded to the element type before P.V
                }
            // Row sum of the rounded probabilities, two per instruction (fp32 accumulation): the
            // denominator then weighs exactly the values the numerator's MFMA sees.
            {
                const X2 ones = {(E)1.f, (E)1.f};
#pragma unroll
                for (int j = 0; j < 4; ++j)
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const X2 pp = {pb[j][2 * e], pb[j][2 * e + 1]};
                        psum = Elem<E>::dot2_acc(pp, ones, psum);
                    }
            }
            l_run += psum;

            // ---- O^T += V^T.P^T ----
            {
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int j = 0; j < 4; ++j)
#pragma unroll
                    for (int db = 0; db < 4; ++db)  // four independent accumulation chains, interleaved
                        oacc[db] = Elem<E>::mfma_32x32x16(vf[j * 4 + db], pb[j], oacc[db]);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    }

    CPMCU_CLOCK(tl_loop_end);
    // ---- the two KV groups meet through LDS ----
    // Each wave keeps half of the output dims of its rows (group 0: d < 64, group 1: d >= 64) and hands the other half
    // to the wave of the other group with the same rows, so that the exchange, the merge and the stores behind it are
    // spread over all eight waves.  The exchange area is the two ring stages the last iteration does not read (the
    // previous iteration's tiles, which every wave has left; no request is in flight into them) and, for (max, sum),
    // the appended-row staging area (last read ahead of a barrier inside the iteration): a wave writes as soon as its
    // own last tile is done, whatever the other group is still doing.
    if constexpr (G == 2) {
        const int i_last = niter > 0 ? 2 * (niter - 1) : 0;
        f32x4* xch = reinterpret_cast<f32x4*>(ring + ((i_last + 2) % kStages) * kStageBytes);  // [wave][8 quads][64 lanes]
        float2* xml = reinterpret_cast<float2*>(vstage);                                        // [wave][64 lanes]
        auto send = [&](auto db0_c) {
            constexpr int DB0 = decltype(db0_c)::value;
#pragma unroll
            for (int db = 0; db < 2; ++db)
#pragma unroll
                for (int rq = 0; rq < 4; ++rq) {
                    f32x4 o;
#pragma unroll
                    for (int e = 0; e < 4; ++e) o[e] = oacc[DB0 + db][rq * 4 + e];
                    xch[(wave * 8 + db * 4 + rq) * 64 + lane] = o;
                }
        };
        if (grp == 0) send(std::integral_constant<int, 2>{});
        else send(std::integral_constant<int, 0>{});
        xml[wave * 64 + lane] = make_float2(m_ref, l_run);
        __syncthreads();
        const int other = wave ^ kRowWaves;  // same rows, other group
        const float2 ml1 = xml[other * 64 + lane];
        const float m_new = fmaxf(m_ref, ml1.x);
        const float m_scaled = (m_new == -INFINITY) ? 0.f : m_new;
        const float a0 = __builtin_amdgcn_exp2f(m_ref - m_scaled);
        const float a1 = __builtin_amdgcn_exp2f(ml1.x - m_scaled);
        auto receive = [&](auto db0_c) {
            constexpr int DB0 = decltype(db0_c)::value;
#pragma unroll
            for (int db = 0; db < 2; ++db)
#pragma unroll
                for (int rq = 0; rq < 4; ++rq) {
                    const f32x4 o = xch[(other * 8 + db * 4 + rq) * 64 + lane];
#pragma unroll
                    for (int e = 0; e < 4; ++e) oacc[DB0 + db][rq * 4 + e] = oacc[DB0 + db][rq * 4 + e] * a0 + o[e] * a1;
                }
        };
        if (grp == 0) receive(std::integral_constant<int, 0>{});
        else receive(std::integral_constant<int, 2>{});
        l_run = l_run * a0 + ml1.y * a1;
        m_ref = m_new;
    }

    CPMCU_CLOCK(tl_groups);
    // oacc[db][r] is O[query qcol][d = db*32 + 8*(r/4) + 4*hf + r%4], unnormalised; with two KV groups a wave now holds
    // the d blocks [2 * grp, 2 * grp + 2) of its rows.
    const float l_tot = l_run + __shfl_xor(l_run, 32);
    // stores db blocks [DB0, DB0 + NDB) of this wave's rows through `put(db, rq, values)`
    auto for_my_blocks = [&](auto&& put) {
        auto run = [&](auto db0_c, auto ndb_c) {
            constexpr int DB0 = decltype(db0_c)::value, NDB = decltype(ndb_c)::value;
#pragma unroll
            for (int db = DB0; db < DB0 + NDB; ++db)
#pragma unroll
                for (int rq = 0; rq < 4; ++rq) put(db, rq, oacc[db]);
        };
        if constexpr (G == 1) run(std::integral_constant<int, 0>{}, std::integral_constant<int, 4>{});
        else if (grp == 0) run(std::integral_constant<int, 0>{}, std::integral_constant<int, 2>{});
        else run(std::integral_constant<int, 2>{}, std::integral_constant<int, 2>{});
    };
    if (p.num_splits == 1) {
        if (!row_ok) return;
        const float inv = (l_tot == 0.f || l_tot != l_tot) ? 1.f : 1.f / l_tot;
        f16* orow = p.out + ((size_t)node * p.Hq + head) * kHeadDim;
        for_my_blocks([&](int db, int rq, const f32x16& acc) {
            X4 o;
#pragma unroll
            for (int e = 0; e < 4; ++e) o[e] = (E)(acc[rq * 4 + e] * inv);
            *reinterpret_cast<X4*>(orow + db * 32 + rq * 8 + hf * 4) = o;
        });
    } else {
        const size_t prow = ((size_t)g * p.num_splits + split) * p.rows_pad + R;
        // Partials leave the kernel normalised (O / l) and rounded to fp16 -- the precision of the
        // final output -- which halves the dominant extra HBM traffic of the split design; (max, l)
        // stay fp32.  The reference keeps fp32 partials; the difference is far inside the tolerance.
        const float inv = (l_tot == 0.f || l_tot != l_tot) ? 0.f : 1.f / l_tot;
        X4* op = reinterpret_cast<X4*>(p.o_part) +
                    ((((size_t)g * p.num_splits + split) * p.num_mtiles + mt) * kRowWaves + rw) * 16 * 64 + lane;
        for_my_blocks([&](int db, int rq, const f32x16& acc) {
            X4 o;
#pragma unroll
            for (int e = 0; e < 4; ++e) o[e] = (E)(acc[rq * 4 + e] * inv);
            if (unit_ctr != nullptr) store_dev64(&op[(db * 4 + rq) * 64], bits_as<uint64_t>(o));
            else __builtin_nontemporal_store(o, &op[(db * 4 + rq) * 64]);  // streamed: nothing left to flush at kernel end
        });
        if (grp == 0 && hf == 0 && row_ok) {
            if (unit_ctr != nullptr) {
                store_dev64(&p.ml_part[prow * 2], (uint64_t)__float_as_uint(m_ref) | ((uint64_t)__float_as_uint(l_tot) << 32));
            } else {
                p.ml_part[prow * 2 + 0] = m_ref;
                p.ml_part[prow * 2 + 1] = l_tot;
            }
        }
#ifdef CPMCU_TIMELINE
        // the records of this workgroup (the stamps sit in registers until here; see timeline.h); records 4..7 stay zero
        // when the merge is a launch of its own
        const auto tl_record = [&]() {
            const int wg = blockIdx.y * gridDim.x + blockIdx.x;
            CPMCU_STAMP_VALUE(g_attn_timeline, wg, 0, tl_start);
            CPMCU_STAMP_VALUE(g_attn_timeline, wg, 1, tl_loop);
            CPMCU_STAMP_VALUE(g_attn_timeline, wg, 2, tl_loop_end);
            CPMCU_STAMP_VALUE(g_attn_timeline, wg, 3, tl_groups);
            CPMCU_STAMP_VALUE(g_attn_timeline, wg, 4, tl_stored);
            CPMCU_STAMP_VALUE(g_attn_timeline, wg, 5, tl_acked);
            CPMCU_STAMP_VALUE(g_attn_timeline, wg, 6, tl_go);
            if (unit_ctr != nullptr) CPMCU_STAMP(g_attn_timeline, wg, 7);
            else CPMCU_STAMP(g_attn_timeline, wg, 4);  // partials issued; the launch ends with them
            CPMCU_STAMP_VALUE(g_attn_timeline, wg, 8, niter);
            CPMCU_STAMP_VALUE(g_attn_timeline, wg, 9, n);
            CPMCU_STAMP_VALUE(g_attn_timeline, wg, 10, split);
            CPMCU_STAMP_VALUE(g_attn_timeline, wg, 11, mt);
            CPMCU_STAMP_VALUE(g_attn_timeline, wg, 12, tl_it1);
            CPMCU_STAMP_VALUE(g_attn_timeline, wg, 13, tl_it2);
            CPMCU_STAMP_VALUE(g_attn_timeline, wg, 14, tl_fix0);
            CPMCU_STAMP_VALUE(g_attn_timeline, wg, 15, tl_fix1);
        };
        if (unit_ctr == nullptr) tl_record();
#endif
        if (unit_ctr == nullptr) return;
        // ---- merge inside the launch ----
        // Every workgroup of the unit (same KV head and M-tile, one per split) announces its partials once they
        // have reached memory; when all have, each merges its share of the unit's 32-row x 4-dim-quad blocks
        // (share s: the blocks b with b % splits == s).
        // The last to arrive never waits; the others wait for it, with a limit -- workgroups that wait for each other
        // must all be resident, which the host checks against the CU count but cannot promise when another launch
        // holds CUs (two such launches on one GPU could wait for each other's unstarted workgroups).  A workgroup
        // whose wait runs out marks its share as abandoned and leaves, which frees its CU; the last to arrive merges
        // the abandoned shares after its own, so the output is complete either way.
        __shared__ int s_merge_go, s_merge_last;
        __shared__ uint32_t s_merge_abandoned;
        CPMCU_CLOCK(tl_stored);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        CPMCU_CLOCK(tl_acked);
        uint32_t* const unit_abandoned = unit_ctr + 1;  // one bit per share; zero between launches (a mark that was made just
                                                        // behind the last arrival's collection is taken back by its maker)
        if (tid == 0) {
            int go = 1, last = 0;
            // The word as this workgroup's arrival found it: the generation of this launch above, the arrivals before it below.
            const uint32_t before = __hip_atomic_fetch_add(unit_ctr, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            const uint32_t full = (before & 0xffff0000u) + (uint32_t)p.num_splits;
            auto all_arrived = [&]() {  // either the full count or, once the last one has moved it on, the next generation
                const uint32_t now = __hip_atomic_load(unit_ctr, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                return now == full || (now & 0xffff0000u) != (before & 0xffff0000u);
            };
            if (before + 1u == full) {
                // last to arrive: full count -> next generation, no arrivals (nobody needs the result of this one)
                __hip_atomic_fetch_add(unit_ctr, 0x10000u - (uint32_t)p.num_splits, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                last = 1;
            } else {
                const unsigned long long t_begin = wall_clock64();
                while (!all_arrived()) {
                    if (wall_clock64() - t_begin >= p.merge_wait_ticks) {
                        // The mark is in memory before this workgroup looks once more: if the others have all arrived by
                        // then, the last of them may have read the marks already, and this workgroup merges its share
                        // itself (twice the same values at worst); if not, the last one will find the mark.
                        // (acquire-release on the mark, acquire on the look that follows: the two stay in this order)
                        (void)__hip_atomic_fetch_or(unit_abandoned, 1u << split, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
                        const uint32_t now = __hip_atomic_load(unit_ctr, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_AGENT);
                        go = (now == full || (now & 0xffff0000u) != (before & 0xffff0000u)) ? 1 : 0;
                        // everyone is there after all: this workgroup merges its share itself and takes its mark back, so that
                        // no mark outlives the launch (if the last arrival has collected it already, the share is merged twice
                        // with the same values)
                        if (go) (void)__hip_atomic_fetch_and(unit_abandoned, ~(1u << split), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        __hip_atomic_fetch_add(&g_attn_report.abandoned, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        break;
                    }
                    __builtin_amdgcn_s_sleep(4);
                }
            }
            s_merge_go = go;
            s_merge_last = last;
        }
        __syncthreads();
        CPMCU_CLOCK(tl_go);
        if (!s_merge_go) return;
        const bool last = s_merge_last != 0;
        // the last one collects the abandoned shares while it merges its own
        uint32_t abandoned = 0;
        if (last && tid == 0) abandoned = __hip_atomic_exchange(unit_abandoned, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const int nblocks = kRowWaves * 16;
        auto merge_share = [&](int share) {
            for (int b = share + p.num_splits * wave; b < nblocks; b += p.num_splits * kWaves)
                combine_block<true, E>(p, g, mt * kRowWaves + (b >> 4), b & 15, lane);
        };
        merge_share(split);
        if (last) {
            if (tid == 0) s_merge_abandoned = abandoned;
            __syncthreads();
            for (uint32_t m = s_merge_abandoned; m != 0; m &= m - 1) merge_share(__builtin_ctz(m));
        }
#ifdef CPMCU_TIMELINE
        tl_record();
#endif
    }
}

// The merge as a launch of its own: one wave per (kv head, 32-row block, quad), in the partial layout's own order.
template <int G, bool ROPE>
__global__ __launch_bounds__(kThreads, 1) void tree_attn_split_kernel(AttnParams p) {
    tree_attn_split_body<G, ROPE, f16>(p);
}
template <int G, bool ROPE>
__global__ __launch_bounds__(kThreads, 1) void tree_attn_split_bf16_kernel(AttnParams p) {
    tree_attn_split_body<G, ROPE, bf16>(p);
}

template <typename E>
__device__ __forceinline__ void tree_attn_combine_body(const AttnParams& p) {
    const int idx = blockIdx.x * 256 + threadIdx.x;
    const int lane = idx & 63;
    const int quad = (idx >> 6) & 15;
    const int nrb = p.rows_pad / kRowsPerWave;  // 32-row blocks per kv head (16 * 64 = 1024 threads each)
    const int grb = idx >> 10;
    if (grb >= p.Hkv * nrb) return;
    combine_block<false, E>(p, grb / nrb, grb % nrb, quad, lane);
}
__global__ __launch_bounds__(256) void tree_attn_combine_kernel(AttnParams p) { tree_attn_combine_body<f16>(p); }
__global__ __launch_bounds__(256) void tree_attn_combine_bf16_kernel(AttnParams p) { tree_attn_combine_body<bf16>(p); }

// Beyond kMergeMaxSplits splits: one workgroup per (kv head, 32-row block, quad) with a wave per batch of 16 splits -- all
// batches in one memory round trip instead of one after the other (128 splits: eight) -- and wave 0 folding the batch
// sums in batch order.
constexpr int kCombineWideWaves = kMaxSplits / kCombineBatch;
template <typename E>
__device__ __forceinline__ void tree_attn_combine_wide_body(const AttnParams& p) {
    __shared__ float s_sum[kCombineWideWaves][6][64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int quad = blockIdx.x & 15;
    const int nrb = p.rows_pad / kRowsPerWave;
    const int grb = blockIdx.x >> 4;
    const CombineWhere<E> w = combine_where<E>(p, grb / nrb, grb % nrb, quad, lane);
    const int nb = (p.num_splits + kCombineBatch - 1) / kCombineBatch;
    CombineSum mine;
    mine.M = -INFINITY;
    mine.L = 0.f;
    mine.acc = f32x4{0.f, 0.f, 0.f, 0.f};
    if (w.valid && wave < nb) mine = combine_batch<false, E>(w, wave * kCombineBatch, p.num_splits);
    if (wave != 0) {
        s_sum[wave][0][lane] = mine.M;
        s_sum[wave][1][lane] = mine.L;
#pragma unroll
        for (int e = 0; e < 4; ++e) s_sum[wave][2 + e][lane] = mine.acc[e];
    }
    __syncthreads();
    if (wave != 0 || !w.valid) return;
    CombineSum t;
    t.M = -INFINITY;
    t.L = 0.f;
    t.acc = f32x4{0.f, 0.f, 0.f, 0.f};
    combine_fold(t, mine);
    for (int b = 1; b < nb; ++b) {
        CombineSum o;
        o.M = s_sum[b][0][lane];
        o.L = s_sum[b][1][lane];
#pragma unroll
        for (int e = 0; e < 4; ++e) o.acc[e] = s_sum[b][2 + e][lane];
        combine_fold(t, o);
    }
    combine_store<E>(p, w, t);
}
__global__ __launch_bounds__(64 * kCombineWideWaves) void tree_attn_combine_wide_kernel(AttnParams p) { tree_attn_combine_wide_body<f16>(p); }
__global__ __launch_bounds__(64 * kCombineWideWaves) void tree_attn_combine_wide_bf16_kernel(AttnParams p) { tree_attn_combine_wide_body<bf16>(p); }

int device_cu_count() {
    static int cus[64] = {0};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 0;
    if (cus[dev] == 0) {
        int v = 0;
        if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 0;
        cus[dev] = v;
    }
    return cus[dev];
}

int choose_splits(int T, int group, int Hkv, int max_kv_len, int G) {
    const int num_mtiles = ceil_div(group * T, rows_per_wg(G));
    const int ntiles = ceil_div(max_kv_len, kTileN);
    // One workgroup per CU.  The grid is (splits x KV heads, padded to a multiple of the XCD count) x M-tiles, and the padding
    // counts: 42 splits of 2 heads on 3 M-tiles are 88 x 3 = 264 workgroups -- too many for the launch to merge itself.
    const int cus = device_cu_count() > 0 ? device_cu_count() : 256;
    int splits = (cus / num_mtiles / kXcds * kXcds) / Hkv;
    if (splits < 1) splits = 1;
    const bool merge = options().attn_merge_in_launch != 0;
    // Between 33 and 63 splits (three M-tiles) a second launch would merge what 32 splits merge in the launch.  24-node tree,
    // us per layer, 42 splits + combine launch against 32 splits: 43.5 / 26.8 at 32K, 55.4 / 34.5 at 48K, 67.5 / 41.9 at
    // 64K, 119 / 79.5 at 128K.
    if (merge && splits > kMergeMaxSplits && splits < 2 * kMergeMaxSplits) splits = kMergeMaxSplits;
    // One or two M-tiles (plain decode, trees of up to 16 nodes) could take 64 or 128 splits; up to about 10K context they
    // do better on at most 32, which the launch can merge itself: 16 while a split still gets about four tiles, 32 beyond.
    // One query, us per layer, 32 splits merged in the launch against 64 with the merge launch (a wave per batch of 16
    // splits): 12.5 / 14.2 at 4K, 14.3 / 14.4 at 8K, 16.2 / 13.9 at 12K, 18.0 / 15.1 at 16K, 21.6 / 17.1 at 24K; 16 nodes:
    // 15.3 / 15.9 at 8K, 17.1 / 17.4 at 12K, 19.0 / 17.7 at 16K.
    constexpr int kShortContextTiles = 160;
    if (merge && splits > kMergeMaxSplits && ntiles <= kShortContextTiles) splits = std::min(kMergeMaxSplits, std::max(16, ntiles / 4));
    // Every split gets at least one tile -- one per KV group when a second launch merges: a launch that merges itself does
    // better on more, shorter splits at short contexts (60-node tree at 512 tokens: 12.7 us on 10 splits, 16.2 on 4).
    const int tile_cap = merge && splits <= kMergeMaxSplits ? ntiles : ntiles / G;
    if (splits > tile_cap) splits = tile_cap > 0 ? tile_cap : 1;
    // More than 64 splits (one M-tile: plain decode, trees of up to 8 nodes) pay for their partials and per-workgroup
    // latencies once every KV group still gets a run of about 3 tiles: one query, 128 against 64 splits, us per layer:
    // 18.6 / 19.0 at 32K, 21.3 / 23.2 at 48K, 23.6 / 27.1 at 64K, 36.4 / 47.5 at 128K (15.8 / 15.1 at 16K).
    if (splits > 64) splits = std::max(64, std::min(splits, ntiles / (G * 3)));
    if (splits > kMaxSplits) splits = kMaxSplits;
    return splits;
}

// KV groups per workgroup.  Per workgroup the 256-row shape runs ntiles / s1 tiles and the two-group shape
// ntiles / (2 s2) iterations of two tiles each, about 1.1-1.2 times as long at long contexts (every tile is fetched
// by twice as many M-tiles), where s1 and s2 are the split counts that fill the CUs with either shape:
//   * s1 beyond what a launch merges itself (one or two 256-row M-tiles, trees of up to 32 nodes; three, up to 48
//     nodes, where the two-group shape has 1.25-1.5 times the splits per tile): two groups.  us per layer, 256-row
//     shape / two groups: 24 nodes 34.6 / 26.9 at 32K, 49.0 / 42.3 at 64K, 82 / 81 at 128K; 40 nodes 40.3 / 33.3 at
//     32K, 67.6 / 56.6 at 64K, 124.5 / 105.7 at 128K; 48 nodes 68.2 / 64.6 at 64K, 127.7 / 122.3 at 128K; 16 nodes or
//     one 74.8 / 62.4 and 73.2 / 55.0 at 128K;
//   * 2 s2 well below s1 (81 to 96 nodes: 8 splits against 20): the 256-row shape from 8K on (96 nodes: 28.7 / 30.8
//     at 8K, 40.0 / 45.9 at 16K, 64.6 / 78.2 at 32K; 21.3 / 19.0 at 2K);
//   * 2 s2 = s1 otherwise: the 256-row shape once every workgroup has a run of at least 16 tiles to amortise its larger
//     split count (twice the partials to merge).  60-node tree (8 units): 30.2 / 27.8 at 16K, 44 / 43 at 32K,
//     75.2 / 77.6 at 64K, 146-152 / 158 at 128K; 128-node tree (16 units): 26.5 / 24.7 at 4K, 49.1 / 49.5 at 16K,
//     82 / 86.5 at 32K, 282 / 300 at 128K; 72 nodes 33.7 / 33.7 at 16K, 53.4 / 55.1 at 32K.
// The option attn_kv_groups (cpmcu_set_option; CPMCU_ATTN_KV_GROUPS=1|2 in the environment at load) overrides the
// choice: tests exercise both shapes.
constexpr int kLongRunTiles = 16;
int splits_that_fill(int T, int group, int Hkv, int G) {
    const int cus = device_cu_count() > 0 ? device_cu_count() : 256;
    const int s = (cus / ceil_div(group * T, rows_per_wg(G)) / kXcds * kXcds) / Hkv;
    return s < 1 ? 1 : s;
}
int choose_groups(int T, int group, int Hkv, int max_kv_len) {
    if (options().attn_kv_groups != 0) return options().attn_kv_groups;
    const int units = ceil_div(group * T, rows_per_wg(1)) * Hkv;
    const int ntiles = ceil_div(max_kv_len, kTileN);
    const int s1 = splits_that_fill(T, group, Hkv, 1), s2 = splits_that_fill(T, group, Hkv, 2);
    if (units < 4 || s1 > kMergeMaxSplits) return 2;
    if (40 * s2 >= 23 * s1) return 2;                       // 2 s2 / s1 >= 1.15
    if (40 * s2 <= 17 * s1) return ntiles >= 128 ? 1 : 2;   // 2 s2 / s1 <= 0.85
    return (long long)ntiles * units >= (long long)kLongRunTiles * 256 ? 1 : 2;
}

// Shape of one attention launch: which kernel shape, how many KV splits and M-tiles.
struct LaunchPlan {
    int span;        // keys the stream can hold: the whole context, or with a window its blocks plus the T new rows
                     // (the window starts on a block boundary at or above P - block_window_size)
    int kv_groups, num_mtiles, num_splits;
    bool merge_in_launch;  // the split workgroups merge their own partials (no combine launch)
};

// Counters of the in-launch merge.  They live in the library (zero when it is loaded, and back at zero arrivals after
// every launch), in blocks handed out per workspace pointer: calls that may overlap use different workspaces and so
// different counters, and nothing has to be cleared or allocated per call.  A block stays with its workspace until
// attention_release_workspace: a captured launch keeps its block's address, so a block is never passed on to another
// workspace.  A launch that cannot have one -- more workspaces than blocks, a first launch under capture -- is merged by
// the combine launch instead.
constexpr int kMergeUnits = 256;    // (KV head, M-tile) units a launch may have on this path
constexpr int kMergeBlocks = 32;    // workspaces with a block per device
__device__ __align__(256) uint32_t g_merge_ctr[kMergeBlocks][kMergeUnits * kMergeUnitWords];

// The split workgroups can merge in the launch when they are all resident at once (one per CU: a workgroup that
// waits for the others must not keep them from starting) and few enough per counter.
bool can_merge_in_launch(int Hkv, int num_mtiles, int num_splits) {
    if (!options().attn_merge_in_launch || num_splits < 2 || num_splits > kMergeMaxSplits) return false;
    if (Hkv * num_mtiles > kMergeUnits) return false;
    return kXcds * ceil_div(num_splits * Hkv, kXcds) * num_mtiles <= device_cu_count();
}

struct MergeState {
    int block = -1;
    bool use_combine = false;  // a wait was abandoned on this device: the workspace's launches are merged by the combine launch
};
std::mutex g_merge_mu;
std::map<std::pair<int, const void*>, MergeState> g_merge_states;
std::vector<int> g_merge_free_blocks[64];
bool g_merge_blocks_listed[64] = {false};
uint32_t* g_merge_ctr_base[64] = {nullptr};

// The counter block of a workspace on the current device; null: the launch has to be merged by the combine launch.
uint32_t* merge_counters_for(const void* workspace, hipStream_t st) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return nullptr;
    std::lock_guard<std::mutex> lock(g_merge_mu);
    auto it = g_merge_states.find({dev, workspace});
    if (it == g_merge_states.end()) {
        if (g_merge_ctr_base[dev] == nullptr) {
            // The address of the counters is looked up once per device, outside any stream capture.
            hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
            if (hipStreamIsCapturing(st, &capturing) != hipSuccess || capturing != hipStreamCaptureStatusNone) {
                (void)hipGetLastError();
                return nullptr;
            }
            void* ptr = nullptr;
            if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(g_merge_ctr)) != hipSuccess) {
                (void)hipGetLastError();
                return nullptr;
            }
            g_merge_ctr_base[dev] = (uint32_t*)ptr;
        }
        if (!g_merge_blocks_listed[dev]) {
            for (int b = kMergeBlocks - 1; b >= 0; --b) g_merge_free_blocks[dev].push_back(b);
            g_merge_blocks_listed[dev] = true;
        }
        if (g_merge_free_blocks[dev].empty()) return nullptr;
        MergeState ns;
        ns.block = g_merge_free_blocks[dev].back();
        g_merge_free_blocks[dev].pop_back();
        it = g_merge_states.emplace(std::make_pair(dev, workspace), ns).first;
    }
    if (it->second.use_combine) return nullptr;
    return g_merge_ctr_base[dev] + (size_t)it->second.block * kMergeUnits * kMergeUnitWords;
}
LaunchPlan plan_launch(int T, int group, int Hkv, int max_kv_len, int block_window_size, int num_splits_override) {
    LaunchPlan pl;
    const int window_blocks = block_window_size / 128;
    pl.span = max_kv_len;
    if (window_blocks > 0 && window_blocks * 128 + T < pl.span) pl.span = window_blocks * 128 + T;
    pl.kv_groups = choose_groups(T, group, Hkv, pl.span);
    pl.num_mtiles = ceil_div(group * T, rows_per_wg(pl.kv_groups));
    pl.num_splits = num_splits_override > 0 ? num_splits_override : choose_splits(T, group, Hkv, pl.span, pl.kv_groups);
    pl.merge_in_launch = can_merge_in_launch(Hkv, pl.num_mtiles, pl.num_splits);
    return pl;
}

}  // namespace
}  // namespace cpmcu

using namespace cpmcu;

// Which kernels an attention call of this shape launches (no launch): names and geometry for reports.
extern "C" int cpmcu_tree_attention_plan(int T, int Hq, int Hkv, int max_kv_len, int with_rope, int block_window_size,
                                         int num_splits_override, char* kernel_names, size_t kernel_names_bytes, int* num_splits,
                                         int* kv_groups, int* num_workgroups) {
    CPMCU_CHECK_ARG(T >= 1 && T <= kMaxTree && Hkv >= 1 && Hq >= Hkv && Hq % Hkv == 0 && max_kv_len >= T, "tree_attention_plan: bad shape");
    const LaunchPlan pl = plan_launch(T, Hq / Hkv, Hkv, max_kv_len, block_window_size, num_splits_override);
    if (kernel_names && kernel_names_bytes > 0)
        snprintf(kernel_names, kernel_names_bytes, "tree_attn_split_kernel<%d,%s>%s", pl.kv_groups, with_rope ? "true" : "false",
                 pl.num_splits <= 1 || pl.merge_in_launch ? "" : pl.num_splits > kMergeMaxSplits ? "+tree_attn_combine_wide_kernel" : "+tree_attn_combine_kernel");
    if (num_splits) *num_splits = pl.num_splits;
    if (kv_groups) *kv_groups = pl.kv_groups;
    if (num_workgroups) *num_workgroups = kXcds * ceil_div(pl.num_splits * Hkv, kXcds) * pl.num_mtiles;
    return CPMCU_OK;
}

namespace cpmcu {
void attention_prepare_workspace(const void* workspace, void* stream) { (void)merge_counters_for(workspace, resolve_stream(stream)); }

// Gives up the counter block of a workspace that is about to be freed (no launch on it may be in flight or captured).
void attention_release_workspace(const void* workspace) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return;
    std::lock_guard<std::mutex> lock(g_merge_mu);
    auto it = g_merge_states.find({dev, workspace});
    if (it == g_merge_states.end()) return;
    g_merge_free_blocks[dev].push_back(it->second.block);
    g_merge_states.erase(it);
}

// The report words of the current device, read without a round trip of their own: `attention_report_enqueue` puts a copy
// into pinned host memory in stream order (call it ahead of a synchronisation of that stream, outside any capture),
// `attention_report_take` looks at that copy afterwards and clears the device words only when something is there.
// After any abandoned wait every workspace of the device goes back to the combine launch.
namespace {
AttnReport* g_report_host[64] = {nullptr};
}
int attention_report_enqueue(hipStream_t st) {
    int dev = 0;
    CPMCU_HIP(hipGetDevice(&dev));
    CPMCU_CHECK_ARG(dev >= 0 && dev < 64, "device index %d outside [0, 64)", dev);
    if (g_report_host[dev] == nullptr) {
        CPMCU_HIP(hipHostMalloc((void**)&g_report_host[dev], sizeof(AttnReport), hipHostMallocDefault));
        *g_report_host[dev] = AttnReport{0, 0u};
    }
    CPMCU_HIP(hipMemcpyFromSymbolAsync(g_report_host[dev], HIP_SYMBOL(g_attn_report), sizeof(AttnReport), 0, hipMemcpyDeviceToHost, st));
    return CPMCU_OK;
}
int attention_report_take(int* bad_length, unsigned int* abandoned) {
    int dev = 0;
    CPMCU_HIP(hipGetDevice(&dev));
    *bad_length = 0;
    *abandoned = 0;
    if (dev < 0 || dev >= 64 || g_report_host[dev] == nullptr) return CPMCU_OK;
    const AttnReport r = *g_report_host[dev];
    if (r.bad_length != 0 || r.abandoned != 0) {
        const AttnReport zero{0, 0u};
        CPMCU_HIP(hipMemcpyToSymbol(HIP_SYMBOL(g_attn_report), &zero, sizeof(zero)));
        *g_report_host[dev] = zero;
        if (r.abandoned != 0) {
            std::lock_guard<std::mutex> lock(g_merge_mu);
            for (auto& kv : g_merge_states)
                if (kv.first.first == dev) kv.second.use_combine = true;
        }
    }
    *bad_length = r.bad_length;
    *abandoned = r.abandoned;
    return CPMCU_OK;
}
// Lets the workspaces of the current device merge inside the launch again (cpmcu_set_option attn_merge_in_launch = 1).
void attention_merge_reenable() {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return;
    std::lock_guard<std::mutex> lock(g_merge_mu);
    for (auto& kv : g_merge_states)
        if (kv.first.first == dev) kv.second.use_combine = false;
}
}  // namespace cpmcu

// 1: a launch on this workspace (outside a stream capture, of a shape that allows it) merges its split partials itself;
// 0: it is merged by the combine launch (no counter block left for the workspace, or the device has seen an abandoned wait).
extern "C" int cpmcu_tree_attention_merge_mode(const void* workspace) {
    int dev = 0;
    if (workspace == nullptr || hipGetDevice(&dev) != hipSuccess) return 0;
    {
        std::lock_guard<std::mutex> lock(g_merge_mu);
        auto it = g_merge_states.find({dev, workspace});
        if (it != g_merge_states.end()) return it->second.use_combine || !options().attn_merge_in_launch ? 0 : 1;
    }
    return merge_counters_for(workspace, nullptr) != nullptr && options().attn_merge_in_launch ? 1 : 0;
}

extern "C" int cpmcu_tree_attention_release_workspace(const void* workspace) {
    CPMCU_CHECK_ARG(workspace, "tree_attention_release_workspace: null pointer argument");
    attention_release_workspace(workspace);
    return CPMCU_OK;
}

extern "C" size_t cpmcu_tree_attention_workspace_bytes(int T, int Hq, int Hkv, int max_kv_len) {
    (void)max_kv_len;
    if (T <= 0 || Hkv <= 0 || Hq <= 0 || Hq % Hkv) return 0;
    const int group = Hq / Hkv;
    const int rows_pad = align_up(group * T, rows_per_wg(1));  // the larger padding of the two kernel shapes
    // sized for the largest split count the library ever picks, so an override fits too
    return align_up((size_t)Hkv * kMaxSplits * rows_pad * kHeadDim * sizeof(f16), 256) +  // normalised fp16 partial outputs
           align_up((size_t)Hkv * kMaxSplits * rows_pad * 2 * sizeof(float), 256);       // (max, sum) per row and split
}

static int tree_attention_impl(const void* q, void* k_pool, void* v_pool,
                               const int32_t* block_table, const int32_t* kv_len, int max_kv_len,
                               const void* k_new, const void* v_new, const float* rope_cos_sin, int block_window_size,
                               const uint64_t* mask, int mask_words, int mask_k_range, int T, int Hq, int Hkv,
                               float scale, void* out, void* workspace, size_t workspace_bytes,
                               int num_splits_override, void* stream) {
    CPMCU_CHECK_ARG(q && k_pool && v_pool && block_table && kv_len && out, "tree_attention: null pointer argument");
    CPMCU_CHECK_ARG(T >= 1 && T <= kMaxTree, "tree_attention: T=%d outside [1, %d]", T, kMaxTree);
    CPMCU_CHECK_ARG(Hkv >= 1 && Hq >= Hkv && Hq % Hkv == 0, "tree_attention: Hq=%d must be a multiple of Hkv=%d", Hq, Hkv);
    CPMCU_CHECK_ARG(max_kv_len >= T, "tree_attention: max_kv_len=%d < T=%d", max_kv_len, T);
    CPMCU_CHECK_ARG(max_kv_len <= (1 << 30), "tree_attention: max_kv_len=%d is beyond the supported context of 2^30 keys", max_kv_len);
    if (mask_k_range == 0 || mask == nullptr) mask_k_range = T;
    CPMCU_CHECK_ARG(mask_k_range >= T && mask_k_range <= kMaxTree && mask_k_range <= max_kv_len,
                    "tree_attention: mask_k_range=%d outside [T=%d, min(%d, max_kv_len)]", mask_k_range, T, kMaxTree);
    CPMCU_CHECK_ARG(mask == nullptr || mask_words == ceil_div(mask_k_range, 64) || (mask_words == 1 && mask_k_range <= 64),
                    "tree_attention: mask_words=%d does not match mask_k_range=%d", mask_words, mask_k_range);
    CPMCU_CHECK_ARG(num_splits_override >= 0 && num_splits_override <= kMaxSplits,
                    "tree_attention: num_splits_override=%d outside [0, %d]", num_splits_override, kMaxSplits);
    CPMCU_CHECK_ARG(block_window_size == 0 || block_window_size >= 128,
                    "tree_attention: block_window_size=%d must be 0 (no window) or at least one block of 128", block_window_size);
    // The reference derives the window's first block per 64-row query block (src/flash_attn/src/flash_blockmask.h:16,32:
    // q_block_idx = m_block + cache length) and never runs a window with more than 64 rows; one start for all rows is
    // what this kernel has, which is the same thing up to 64 rows.
    CPMCU_CHECK_ARG(block_window_size == 0 || T <= 64, "tree_attention: a block window with T=%d rows is not supported (at most 64)", T);
    const int group = Hq / Hkv;
    AttnParams p;
    p.q = (const f16*)q;
    p.k_pool = (const f16*)k_pool;
    p.v_pool = (const f16*)v_pool;
    p.block_table = block_table;
    p.kv_len = kv_len;
    CPMCU_CHECK_ARG((k_new == nullptr) == (v_new == nullptr), "tree_attention: k_new and v_new must be given together");
    p.k_new = (const f16*)k_new;
    p.v_new = (const f16*)v_new;
    p.rope = (const float2*)rope_cos_sin;
    p.k_pool_w = (f16*)k_pool;
    p.v_pool_w = (f16*)v_pool;
    p.mask = mask;
    p.mask_words = mask ? mask_words : 0;
    p.mask_k_range = mask_k_range;
    p.T = T;
    p.Hq = Hq;
    p.Hkv = Hkv;
    p.group = group;
    auto log2_or_minus1 = [](int v) {
        int sft = 0;
        while ((1 << sft) < v) ++sft;
        return (1 << sft) == v ? sft : -1;
    };
    p.group_shift = log2_or_minus1(group);
    p.hkv_shift = log2_or_minus1(Hkv);
    p.window_blocks = block_window_size / 128;
    const LaunchPlan plan = plan_launch(T, group, Hkv, max_kv_len, block_window_size, num_splits_override);
    const int span = plan.span;
    const int G = plan.kv_groups;
    p.num_mtiles = plan.num_mtiles;
    p.rows_pad = p.num_mtiles * rows_per_wg(G);
    p.num_splits = plan.num_splits;
    CPMCU_CHECK_ARG(p.num_splits <= kMaxSplits, "tree_attention: max_kv_len=%d is beyond the supported context", max_kv_len);
    p.ntiles_max = ceil_div(span, kTileN);
    p.table_pages = ceil_div(max_kv_len, kPage);
    p.max_kv_len = max_kv_len;
    p.scale_log2 = scale * 1.4426950408889634f;
    p.out = (f16*)out;
    hipStream_t st = resolve_stream(stream);
    p.o_part = nullptr;
    p.ml_part = nullptr;
    p.merge_ctr = nullptr;
    p.merge_wait_ticks = 0;
    if (p.num_splits > 1) {
        const size_t o_bytes = align_up((size_t)Hkv * p.num_splits * p.rows_pad * kHeadDim * sizeof(f16), 256);
        const size_t ml_bytes = (size_t)Hkv * p.num_splits * p.rows_pad * 2 * sizeof(float);
        CPMCU_CHECK_ARG(workspace && workspace_bytes >= o_bytes + ml_bytes,
                        "tree_attention: workspace of %zu bytes needed, %zu given", o_bytes + ml_bytes, workspace_bytes);
        p.o_part = (float*)workspace;
        p.ml_part = (float*)((char*)workspace + o_bytes);
        if (plan.merge_in_launch) p.merge_ctr = merge_counters_for(workspace, st);
        p.merge_wait_ticks = (uint32_t)options().attn_merge_wait_us * 100u;
    }
    const int nsh = p.num_splits * Hkv;
    const dim3 grid(kXcds * ceil_div(nsh, kXcds), p.num_mtiles);
    const bool is_bf16 = options().dtype == 1;
    if (is_bf16) {
        if (p.rope != nullptr) {
            if (G == 1) hipLaunchKernelGGL((tree_attn_split_bf16_kernel<1, true>), grid, dim3(kThreads), 0, st, p);
            else hipLaunchKernelGGL((tree_attn_split_bf16_kernel<2, true>), grid, dim3(kThreads), 0, st, p);
        } else {
            if (G == 1) hipLaunchKernelGGL((tree_attn_split_bf16_kernel<1, false>), grid, dim3(kThreads), 0, st, p);
            else hipLaunchKernelGGL((tree_attn_split_bf16_kernel<2, false>), grid, dim3(kThreads), 0, st, p);
        }
    } else if (p.rope != nullptr) {
        if (G == 1) hipLaunchKernelGGL((tree_attn_split_kernel<1, true>), grid, dim3(kThreads), 0, st, p);
        else hipLaunchKernelGGL((tree_attn_split_kernel<2, true>), grid, dim3(kThreads), 0, st, p);
    } else {
        if (G == 1) hipLaunchKernelGGL((tree_attn_split_kernel<1, false>), grid, dim3(kThreads), 0, st, p);
        else hipLaunchKernelGGL((tree_attn_split_kernel<2, false>), grid, dim3(kThreads), 0, st, p);
    }
    CPMCU_LAUNCH_CHECK();
    if (p.num_splits > 1 && p.merge_ctr == nullptr) {
        const int waves_total = Hkv * (p.rows_pad / kRowsPerWave) * 16;  // one per (kv head, 32-row block, quad)
        if (p.num_splits > kMergeMaxSplits) {
            const dim3 block(64 * ceil_div(p.num_splits, kCombineBatch));
            if (is_bf16) hipLaunchKernelGGL(tree_attn_combine_wide_bf16_kernel, dim3(waves_total), block, 0, st, p);
            else hipLaunchKernelGGL(tree_attn_combine_wide_kernel, dim3(waves_total), block, 0, st, p);
        } else if (is_bf16) {
            hipLaunchKernelGGL(tree_attn_combine_bf16_kernel, dim3(ceil_div(waves_total * 64, 256)), dim3(256), 0, st, p);
        } else {
            hipLaunchKernelGGL(tree_attn_combine_kernel, dim3(ceil_div(waves_total * 64, 256)), dim3(256), 0, st, p);
        }
        CPMCU_LAUNCH_CHECK();
    }
    return CPMCU_OK;
}

extern "C" int cpmcu_tree_attention(const void* q, void* k_pool, void* v_pool,
                                    const int32_t* block_table, const int32_t* kv_len, int max_kv_len,
                                    const void* k_new, const void* v_new,
                                    const uint64_t* mask, int mask_words, int mask_k_range, int T, int Hq, int Hkv,
                                    float scale, void* out, void* workspace, size_t workspace_bytes,
                                    int num_splits_override, void* stream) {
    return tree_attention_impl(q, k_pool, v_pool, block_table, kv_len, max_kv_len, k_new, v_new, nullptr, 0, mask, mask_words,
                               mask_k_range, T, Hq, Hkv, scale, out, workspace, workspace_bytes, num_splits_override, stream);
}

extern "C" int cpmcu_tree_attention_rope(const void* q, void* k_pool, void* v_pool,
                                         const int32_t* block_table, const int32_t* kv_len, int max_kv_len,
                                         const void* k_new, const void* v_new, const float* rope_cos_sin,
                                         const uint64_t* mask, int mask_words, int mask_k_range, int T, int Hq, int Hkv,
                                         float scale, void* out, void* workspace, size_t workspace_bytes,
                                         int num_splits_override, void* stream) {
    CPMCU_CHECK_ARG(rope_cos_sin, "tree_attention_rope: null rotary table");
    return tree_attention_impl(q, k_pool, v_pool, block_table, kv_len, max_kv_len, k_new, v_new, rope_cos_sin, 0, mask, mask_words,
                               mask_k_range, T, Hq, Hkv, scale, out, workspace, workspace_bytes, num_splits_override, stream);
}

extern "C" int cpmcu_tree_attention_window(const void* q, void* k_pool, void* v_pool,
                                           const int32_t* block_table, const int32_t* kv_len, int max_kv_len,
                                           const void* k_new, const void* v_new, const float* rope_cos_sin,
                                           int block_window_size,
                                           const uint64_t* mask, int mask_words, int mask_k_range, int T, int Hq, int Hkv,
                                           float scale, void* out, void* workspace, size_t workspace_bytes,
                                           int num_splits_override, void* stream) {
    CPMCU_CHECK_ARG(block_window_size >= 0, "tree_attention_window: block_window_size=%d is negative", block_window_size);
    return tree_attention_impl(q, k_pool, v_pool, block_table, kv_len, max_kv_len, k_new, v_new, rope_cos_sin, block_window_size,
                               mask, mask_words, mask_k_range, T, Hq, Hkv, scale, out, workspace, workspace_bytes,
                               num_splits_override, stream);
}

namespace cpmcu {
namespace {

// cos / sin of every (row position, frequency) pair, exactly the values rotary_embedding_kernel
// (src/model/rotary.cuh:11-17) computes per element: freq = float(pos) * inv_freq[col].
__global__ void rope_table_kernel(const int32_t* pos, const float* inv_freq, int half_dim, float2* out) {
    const int t = blockIdx.x;
    const float p = (float)pos[t];
    for (int col = threadIdx.x; col < half_dim; col += blockDim.x) {
        const float freq = p * inv_freq[col];
        out[(size_t)t * half_dim + col] = make_float2(cosf(freq), sinf(freq));
    }
}

// rotary_embedding_kernel, src/model/rotary.cuh:7-34, from a table: in place on q [T][Hq][128] and k [T][Hkv][128].
template <typename E>
__global__ __launch_bounds__(256) void rope_apply_kernel(const float2* table, int Hq, int Hkv, E* q, E* k) {
    constexpr int half = kHeadDim / 2;
    const int t = blockIdx.x;
    const float2* cs = table + (size_t)t * half;
    for (int i = threadIdx.x; i < (Hq + Hkv) * half; i += 256) {
        const int row = i / half, col = i % half;
        E* x = row < Hq ? q + ((size_t)t * Hq + row) * kHeadDim : k + ((size_t)t * Hkv + (row - Hq)) * kHeadDim;
        E a = x[col], b = x[col + half];
        rotate_pair(a, b, cs[col]);
        x[col] = a;
        x[col + half] = b;
    }
}

}  // namespace
}  // namespace cpmcu

extern "C" int cpmcu_rope_table(const int32_t* position_ids, const float* inv_freq, int T, float* cos_sin, void* stream) {
    CPMCU_CHECK_ARG(position_ids && inv_freq && cos_sin, "rope_table: null pointer argument");
    CPMCU_CHECK_ARG(T >= 1, "rope_table: T=%d", T);
    hipLaunchKernelGGL(rope_table_kernel, dim3(T), dim3(64), 0, resolve_stream(stream), position_ids, inv_freq, kHeadDim / 2,
                       (float2*)cos_sin);
    CPMCU_LAUNCH_CHECK();
    return CPMCU_OK;
}

extern "C" int cpmcu_rope_apply(const float* cos_sin, int T, int Hq, int Hkv, void* q, void* k, void* stream) {
    CPMCU_CHECK_ARG(cos_sin && q && k, "rope_apply: null pointer argument");
    CPMCU_CHECK_ARG(T >= 1 && Hq >= 1 && Hkv >= 1, "rope_apply: T=%d Hq=%d Hkv=%d", T, Hq, Hkv);
    if (options().dtype == 1)
        hipLaunchKernelGGL(rope_apply_kernel<bf16>, dim3(T), dim3(256), 0, resolve_stream(stream), (const float2*)cos_sin, Hq, Hkv, (bf16*)q, (bf16*)k);
    else
        hipLaunchKernelGGL(rope_apply_kernel<f16>, dim3(T), dim3(256), 0, resolve_stream(stream), (const float2*)cos_sin, Hq, Hkv, (f16*)q, (f16*)k);
    CPMCU_LAUNCH_CHECK();
    return CPMCU_OK;
}

CPMCU_TIMELINE_READER(cpmcu_timeline_read_attention, cpmcu::g_attn_timeline)
