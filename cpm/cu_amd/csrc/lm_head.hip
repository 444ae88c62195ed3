// Skinny lm_head GEMMs for gfx950 (MI355X): logits[n, V] = hidden[n, H] . W[V, H]^T with
// n <= 128 rows, fp16 in, fp32 accumulate, streaming W from HBM exactly once.
//
// Two epilogues share one kernel:
//   * STATS  -- FR-Spec draft head (src/model/linear.cuh:8-37,73-79 as called from
//     src/model/minicpm4/minicpm4_eagle.cuh:320,366): writes the fp16 logits and, per
//     workgroup, partial (max, sum exp) of every hidden row for the log-softmax that
//     follows (src/model/eagle.cuh:29-89).
//   * ARGMAX -- target head (src/model/linear.cuh:82-101, fp16 pre-scale by head_scale) with
//     the arg-max of cpmcu/speculative/tree_drafter.py:153,233 fused: per workgroup the best
//     (value, lowest index) of every hidden row; logits are materialised only on request.
//
// The path is HBM-bound (n flop per byte of W), so the design is about keeping many 16-byte
// loads of W in flight per CU, not about MFMA peak:
//   * one persistent workgroup of 8 waves per CU; every wave owns whole 16-row blocks of W and
//     the full K range, so nothing is reduced across waves inside the loop;
//   * W goes HBM -> registers directly as the A operand of v_mfma_f32_16x16x32_f16.  In the tiled
//     layout (cpmcu_head_weight_tile: [V/16][H/32][64 lanes][8 halves]) every wave instruction
//     reads one contiguous KB and consecutive k-steps are consecutive in memory; the row-major
//     layout is read as lane = (row % 16, k-group), 4 lanes per 64 contiguous bytes of a row;
//   * the hidden rows are the B operand, staged in LDS: resident for the whole K range with up
//     to 16 rows on the row-major path (head_gemm_kernel), otherwise walked in K chunks that are
//     brought in by direct-to-LDS loads, double buffered, in the OUTER loop, with one accumulator
//     set per row block of a sweep (head_gemm_chunked_kernel); tiled weights of at least one full pass run
//     head_gemm_stream_kernel, which keeps the W stream in a register ring refilled fragment by fragment
//     (one to four full passes per wave; more workgroups than CUs for larger vocabularies);
//   * when the row blocks do not divide evenly over the wave slots, the blocks of the partly
//     filled last pass are dealt round-robin to the workgroups and several waves share each of
//     them, every one taking a subset of the K chunks; their partial sums meet in LDS.
#include <map>
#include <mutex>
#include <tuple>
#include <type_traits>
#include <vector>

#include "common.h"
#include "internal.h"
#include "timeline.h"
#include "topk_keys.h"

namespace cpmcu {
namespace {

constexpr int kHeadWaves = 8;
constexpr int kHeadThreads = kHeadWaves * 64;

struct HeadParams {
    const f16* hidden;
    const f16* w;
    int n, V, H;
    int kc;       // K chunk held in one LDS buffer
    int nch;      // H / kc
    int npasses;  // row-block passes per workgroup
    // Shared last pass (chunked kernel, single sweep): when the row blocks do not fill the last pass, its
    // blocks are dealt to the workgroups round-robin and each is worked on by several waves, every one
    // taking a subset of the K chunks, so that all waves carry the same load.  full_passes = npasses - 1
    // complete passes, rem_blocks = row blocks left for the last one; 0 = plain mapping.
    int full_passes;
    int rem_blocks;
    int last_share;  // streaming kernel: waves that share one row block of the last pass (power of two)
    int apply_scale;
    float head_scale;
    int mode;
    int w_tiled;  // W is stored as MFMA operand tiles: [16-row block][32-column step][lane][8 halves]
    f16* logits;          // [n][V] or null
    float* part_a;        // STATS: max   | ARGMAX: best value      [grid][NB*16]
    float* part_b;        // STATS: sum   | ARGMAX: best index (int) [grid][NB*16]
};

template <int NB>
struct HeadCfg {
    static constexpr int kKcMax = 2048 / NB;             // halves of K per hidden row per buffer
    static constexpr int kGroupK = NB <= 4 ? 512 : 256;  // K covered by one prefetch group
    static constexpr int kDepth = kGroupK / 32;          // 16-byte loads in flight per lane
    static constexpr int kLdsRowMax = kKcMax * 2 + 16;   // bytes, padded: conflict-free b128 reads
    static constexpr int kLdsBuf = NB * 16 * kLdsRowMax;
    static constexpr int kStage = 8;                     // 16-byte staging registers per thread
};

// ---- FR-Spec head with its log-softmax / top-k / id map-back in the same launch -------------------------------------
// (src/model/minicpm4/minicpm4_eagle.cuh:366-372: Linear::prefill, log_softmax, TopK::prefill, remap as four+ launches.)
// Every GEMM workgroup ranks its own logits of a hidden row first (the k..16 largest as (value, index) keys, ties to
// the lower index) and publishes them, with the row's partial (max, sum exp), as self-validating 64-bit words: each
// word carries the generation of its row, is written by one device-scope store and read by one device-scope load, so
// a reader that sees the generation sees the payload -- no fence, no acknowledged store, no arrival counter between
// producer and consumer.  The first n workgroups to finish (a ticket each) become the finishers of one row each:
// they poll that row's words of all workgroups, rank the few candidates at or above a bound exactly as the row
// kernel of topk.hip does, and write the outputs.  What the words cannot decide -- a workgroup with more candidates
// than slots (rows dominated by one value) -- is redone from the logits in memory, which every workgroup marks
// complete after its stores have been acknowledged.
constexpr int kFuseStates = 8;      // (workspace, grid) pairs per device that can have a launch in flight or captured
constexpr int kFuseMaxGrid = 256;
constexpr int kFuseRows = 16;
constexpr int kFuseSlots = 16;
constexpr int kFuseCap = kHeadThreads;  // candidate keys a finisher ranks
constexpr int kFuseIdBits = 20;
constexpr uint32_t kFuseCandTagMask = 0x7FFFFu;

struct HeadFuseState {
    unsigned long long tickets;  // never reset: a launch of G workgroups takes G of them, ticket % G is the order of finishing
    uint32_t gen[kFuseRows];     // generation of each hidden row's words; advanced by the row's finisher
    uint32_t pad[46];
    uint64_t done[kFuseMaxGrid];                        // generation of row 0 | this workgroup's logits are in memory
    uint64_t stats[kFuseRows][kFuseMaxGrid];            // tag:16 | max z (element bits):16 | sum exp (fp32 bits, sign = wide ids)
    uint64_t cand[kFuseRows][kFuseMaxGrid][kFuseSlots];  // tag:19 | ordered image of z:16 | index within the workgroup:9 | token id:20
};
static_assert(sizeof(HeadFuseState) % 256 == 0, "states stay 256-byte aligned");
__device__ __attribute__((aligned(256))) HeadFuseState g_head_fuse[kFuseStates];
struct HeadFuseReport {
    unsigned int timeouts;    // finishers whose wait ran out (their rows were not written)
    unsigned int slow_rows;   // rows redone from the logits in memory
    unsigned int fused_rows;  // rows finished from the published candidates
};
__device__ HeadFuseReport g_head_fuse_report;

// Timeline records of the streaming kernels (timeline.h): 0 start, 1 wave 0 out of the K loop, 2 full passes folded,
// 3 last pass folded, 4 workgroup's partials / statistics out, 8..15 each wave out of the K loop; one-launch FR-Spec
// form: 5 keys published, 6 stores acknowledged, 7 place known (note 12: place + 1), finishers: 9 all words seen,
// 10 bound known, 11 candidates listed, 13 row written (note 14: candidates).
CPMCU_TIMELINE_STORAGE(g_head_timeline)

struct FuseParams {
    HeadFuseState* st;
    int top;
    const int32_t* remap;
    uint16_t* val;
    int32_t* pos;
    int32_t* ids;
    float* row_stats;
    uint32_t wait_ticks;  // longest wait of a finisher, in ticks of the 100 MHz wall clock
};

__device__ inline uint64_t fuse_load(const uint64_t* p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ inline void fuse_store(uint64_t* p, uint64_t v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
// A workgroup publishes at least this many keys of a row (all it has, if fewer): with small k a few more than k, so that
// a workgroup whose every published key is a candidate -- the case the finisher cannot decide -- stays rare.
__device__ inline int fuse_publish_min(int top) { return top > 8 ? top : 8; }
__device__ inline uint16_t image_to_bits(uint32_t o) { return (uint16_t)((o & 0x8000u) ? (o ^ 0x8000u) : (o ^ 0xFFFFu)); }

// Folds the part of one finished 16-row block of W that belongs to hidden-row block nb (acc[r] <-> vocab row vrow0 + r,
// hidden row nb*16 + l16) into the lane's running epilogue state and writes its logits when asked to.
// ASCENDING: the caller hands a lane its vocabulary rows in ascending order and has preset the state to (-inf, the
// lane's first row), so "lowest index among equals" needs no comparison of indices here: a later equal value never
// replaces an earlier one.  (Five vector instructions per value instead of nine in the arg-max-only case, which is
// what the verify step's 60-row head spends its last microseconds on.)
template <typename E, bool ASCENDING>
__device__ inline void head_epilogue_block(const HeadParams& p, const f32x4& acc, int nb, int vrow0, int l16, float& ea, float& eb) {
    const int V = p.V;
    if (p.mode == kHeadModeArgmax && p.logits == nullptr) {
        // The verify step's case (arg-max only), without a branch per value: the comparisons below as selects.
        const bool row_in = nb * 16 + l16 < p.n;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const float x = (float)(E)acc[r];
            const int idx = vrow0 + r;
            const bool better = ASCENDING ? x > ea : (x > ea || (x == ea && idx < __float_as_int(eb)));
            const bool take = row_in && idx < V && better;
            ea = take ? x : ea;
            eb = take ? __int_as_float(idx) : eb;
        }
        return;
    }
    const int hrow = nb * 16 + l16;
    E z[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) z[r] = (E)acc[r];
    if (hrow < p.n) {
        if (p.logits) {
            E* dst = reinterpret_cast<E*>(p.logits) + (size_t)hrow * V + vrow0;
            if ((V & 3) == 0 && vrow0 + 3 < V) {
                typename Elem<E>::x4 zz;
#pragma unroll
                for (int r = 0; r < 4; ++r) zz[r] = z[r];
                *reinterpret_cast<typename Elem<E>::x4*>(dst) = zz;
            } else {
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    if (vrow0 + r < V) dst[r] = z[r];
            }
        }
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            if (vrow0 + r >= V) continue;
            const float x = (float)z[r];
            if (p.mode == kHeadModeStats) {
                if (x == -INFINITY) continue;  // contributes exp(-inf) = 0
                if (x > ea) {
                    eb = eb * __expf(ea - x) + 1.f;
                    ea = x;
                } else {
                    eb += __expf(x - ea);
                }
            } else {
                const int idx = vrow0 + r;
                const int bidx = __float_as_int(eb);
                if (x > ea || (!ASCENDING && x == ea && idx < bidx)) {
                    ea = x;
                    eb = __int_as_float(idx);
                }
            }
        }
    }
}
template <int NB, typename E, bool ASCENDING = false>
__device__ inline void head_epilogue(const HeadParams& p, const f32x4 (&acc)[NB], int vrow0, int l16, float (&ea)[NB], float (&eb)[NB]) {
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) head_epilogue_block<E, ASCENDING>(p, acc[nb], nb, vrow0, l16, ea[nb], eb[nb]);
}

// Reduces the epilogue state over the lanes that share a hidden row, then over the waves, and writes
// the workgroup's partials.
template <int NB, typename Write>
__device__ inline void head_finish_with(const HeadParams& p, float (&ea)[NB], float (&eb)[NB], float (*red_a)[NB * 16], float (*red_b)[NB * 16],
                                        int tid, int wave, int lane, Write write) {
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
#pragma unroll
        for (int off = 16; off <= 32; off <<= 1) {
            const float oa = __shfl_xor(ea[nb], off);
            const float ob = __shfl_xor(eb[nb], off);
            if (p.mode == kHeadModeStats) {
                const float m = fmaxf(ea[nb], oa);
                const float s = (m == -INFINITY) ? 0.f : eb[nb] * __expf(ea[nb] - m) + ob * __expf(oa - m);
                ea[nb] = m;
                eb[nb] = s;
            } else {
                if (oa > ea[nb] || (oa == ea[nb] && __float_as_int(ob) < __float_as_int(eb[nb]))) {
                    ea[nb] = oa;
                    eb[nb] = ob;
                }
            }
        }
        if (lane < 16) {
            red_a[wave][nb * 16 + lane] = ea[nb];
            red_b[wave][nb * 16 + lane] = eb[nb];
        }
    }
    __syncthreads();
    if (tid < NB * 16) {
        float a = red_a[0][tid], b = red_b[0][tid];
        for (int w = 1; w < kHeadWaves; ++w) {
            const float oa = red_a[w][tid], ob = red_b[w][tid];
            if (p.mode == kHeadModeStats) {
                const float m = fmaxf(a, oa);
                b = (m == -INFINITY) ? 0.f : b * __expf(a - m) + ob * __expf(oa - m);
                a = m;
            } else if (oa > a || (oa == a && __float_as_int(ob) < __float_as_int(b))) {
                a = oa;
                b = ob;
            }
        }
        write(tid, a, b);
    }
}
template <int NB>
__device__ inline void head_finish(const HeadParams& p, float (&ea)[NB], float (&eb)[NB], float (*red_a)[NB * 16], float (*red_b)[NB * 16],
                                   int tid, int wave, int lane, int c) {
    head_finish_with<NB>(p, ea, eb, red_a, red_b, tid, wave, lane, [&](int row, float a, float b) {
        p.part_a[(size_t)c * (NB * 16) + row] = a;
        p.part_b[(size_t)c * (NB * 16) + row] = b;
    });
}

template <int NB, typename E>
__device__ __forceinline__ void head_gemm_body(const HeadParams& p) {
    typedef typename Elem<E>::x8 X8;
    using C = HeadCfg<NB>;
    constexpr int PD = C::kDepth;
    constexpr int GK = C::kGroupK;
    __shared__ __attribute__((aligned(16))) char lds[2 * C::kLdsBuf];
    __shared__ float red_a[kHeadWaves][NB * 16];
    __shared__ float red_b[kHeadWaves][NB * 16];

    const int tid = threadIdx.x;
    const int wave = tid >> 6;
    const int lane = tid & 63;
    const int l16 = lane & 15;
    const int kgp = lane >> 4;  // k-group of this lane inside a 32-wide k-step
    const int G = gridDim.x;
    const int c = blockIdx.x;
    const int H = p.H, V = p.V, kc = p.kc, nch = p.nch;
    const int lds_row = kc * 2 + 16;
    const bool resident = nch <= 2;
    const int gpp = H / GK;  // prefetch groups per pass
    const int total = p.npasses * gpp;
    const int total_chunks = p.npasses * nch;
    // Every workgroup (and, when all of hidden is LDS-resident, every wave) walks K from a different
    // starting chunk.  All rows of W are H*2 bytes apart, so waves that swept K in lockstep would
    // keep hitting addresses with the same low bits -- the same few HBM channels -- at any instant.
    const int rotc = resident ? 0 : c % nch;
    const int rotg = resident ? (c * kHeadWaves + wave) % gpp : rotc * (kc / GK);
    const E sc = (E)p.head_scale;

    // ---- hidden staging helpers ----
    const int chunks16 = NB * 16 * kc / 8;  // 16-byte pieces per K chunk
    X8 stage[C::kStage];
    auto stage_load = [&](int hchunk) {
#pragma unroll
        for (int s = 0; s < C::kStage; ++s) {
            const int i = tid + s * kHeadThreads;
            if (i < chunks16) {
                const int row = i / (kc / 8);
                const int col = (i % (kc / 8)) * 8;
                X8 x;
                if (row < p.n) {
                    x = *reinterpret_cast<const X8*>(p.hidden + (size_t)row * H + (size_t)hchunk * kc + col);
                    if (p.apply_scale) {
#pragma unroll
                        for (int e = 0; e < 8; ++e) x[e] = (E)((float)x[e] * (float)sc);
                    }
                } else {
#pragma unroll
                    for (int e = 0; e < 8; ++e) x[e] = (E)0.f;
                }
                stage[s] = x;
            }
        }
    };
    auto stage_store = [&](int buf) {
#pragma unroll
        for (int s = 0; s < C::kStage; ++s) {
            const int i = tid + s * kHeadThreads;
            if (i < chunks16) {
                const int row = i / (kc / 8);
                const int col = (i % (kc / 8)) * 8;
                *reinterpret_cast<X8*>(lds + (size_t)buf * C::kLdsBuf + row * lds_row + col * 2) = stage[s];
            }
        }
    };

    // ---- W prefetch: group `it` = (pass, k-group) of this wave's row block ----
    const int arow_lane = l16;
    auto row_block = [&](int pass) { return (pass * kHeadWaves + wave) * G + c; };
    auto load_group = [&](int it, X8* buf) {
        const int pass = it / gpp;
        const int k0 = ((it % gpp + rotg) % gpp) * GK;
        if (p.w_tiled) {  // one contiguous KB per instruction, consecutive steps consecutive in memory
            int rb = row_block(pass);
            rb = rb * 16 < V ? rb : (V - 1) / 16;
            const f16* src = p.w + ((size_t)rb * (H / 32) + k0 / 32) * 512 + lane * 8;
#pragma unroll
            for (int ks = 0; ks < PD; ++ks) buf[ks] = __builtin_nontemporal_load(reinterpret_cast<const X8*>(src + ks * 512));
            return;
        }
        int row = row_block(pass) * 16 + arow_lane;
        row = row < V ? row : V - 1;  // clamp: rows past the end are computed and discarded
        const f16* src = p.w + (size_t)row * H + k0 + kgp * 8;
#pragma unroll
        for (int ks = 0; ks < PD; ++ks) buf[ks] = __builtin_nontemporal_load(reinterpret_cast<const X8*>(src + ks * 32));
    };

    f32x4 acc[NB];
    // running epilogue state of this lane, per n-block: hidden row nb*16 + l16
    float ea[NB], eb[NB];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
        ea[nb] = -INFINITY;                      // running max / best value
        eb[nb] = p.mode == kHeadModeStats ? 0.f : __int_as_float(0x7fffffff);  // running sum / best index
    }

    auto epilogue = [&](int pass) { head_epilogue<NB, E>(p, acc, row_block(pass) * 16 + kgp * 4, l16, ea, eb); };

    // ---- prologue: hidden into LDS ----
    if (resident) {
        for (int ch = 0; ch < nch; ++ch) {
            stage_load(ch);
            stage_store(ch);
        }
        __syncthreads();
    } else {
        stage_load(rotc);
        stage_store(0);
    }

    auto compute_group = [&](int it, const X8* buf) {
        const int pass = it / gpp;
        const int kg = it % gpp;                     // position in this wave's K walk
        const int k0 = ((kg + rotg) % gpp) * GK;     // actual K offset (rotated by whole chunks)
        const int chunk = (kg * GK) / kc;            // sequential chunk number of the walk
        const int koff = k0 % kc;
        const int cglobal = pass * nch + chunk;
        int lbuf;
        if (resident) {
            lbuf = k0 / kc;
        } else {
            if (koff == 0) {
                __syncthreads();  // chunk `cglobal` visible; everyone is done with the other buffer
                if (cglobal + 1 < total_chunks) stage_load(((cglobal + 1) % nch + rotc) % nch);
            }
            lbuf = cglobal & 1;
        }
        if (kg == 0) {
#pragma unroll
            for (int nb = 0; nb < NB; ++nb)
#pragma unroll
                for (int r = 0; r < 4; ++r) acc[nb][r] = 0.f;
        }
        const char* brow = lds + (size_t)lbuf * C::kLdsBuf + l16 * lds_row + (koff + kgp * 8) * 2;
#pragma unroll
        for (int ks = 0; ks < PD; ++ks) {
#pragma unroll
            for (int nb = 0; nb < NB; ++nb) {
                const X8 b = *reinterpret_cast<const X8*>(brow + nb * 16 * lds_row + ks * 64);
                acc[nb] = Elem<E>::mfma_16x16x32(buf[ks], b, acc[nb]);
            }
        }
        if (!resident && koff + GK == kc) {
            if (cglobal + 1 < total_chunks) stage_store((cglobal + 1) & 1);
        }
        if (kg == gpp - 1) epilogue(pass);
    };

    X8 buf_a[PD], buf_b[PD];
    if (total > 0) load_group(0, buf_a);
    for (int it = 0; it < total; it += 2) {
        if (it + 1 < total) load_group(it + 1, buf_b);
        compute_group(it, buf_a);
        if (it + 1 < total) {
            if (it + 2 < total) load_group(it + 2, buf_a);
            compute_group(it + 1, buf_b);
        }
    }

    head_finish<NB>(p, ea, eb, red_a, red_b, tid, wave, lane, c);
}

// More than 16 hidden rows do not fit LDS for the whole K range.  This kernel walks K in chunks in the
// OUTER loop: a chunk of all hidden rows (64 KB) is brought into LDS by direct-to-LDS loads, double
// buffered, and every wave then streams that K range of each of its row blocks of W, keeping one
// accumulator set per row block (NP row blocks per sweep over K).  The workgroup synchronises once
// per chunk, not once per (row block, chunk), so the waves' W streams run free in between.
//   LDS layout of a chunk: [hidden row][KC halves], unpadded; the 16-byte piece index is XORed with
//   row % 16 (applied through the global address each DMA lane fetches), which makes the B-operand
//   reads (16 rows x one piece per 16 lanes) conflict-free.
template <int NB, int NP, int KC, int NBUF, typename E>  // KC = halves of K per chunk, NBUF = W register buffers
__device__ __forceinline__ void head_gemm_chunked_body(const HeadParams& p) {
    typedef typename Elem<E>::x8 X8;
    constexpr int PD = KC / 32;              // 16-byte W loads in flight per lane and buffer
    constexpr int ROWB = KC * 2;
    constexpr int BUF = NB * 16 * ROWB;
    constexpr int PR = KC / 8;               // 16-byte pieces per hidden row chunk
    constexpr int NINST = BUF / 1024 / kHeadWaves;  // 1 KB DMA instructions per wave and chunk
    static_assert(NP % NBUF == 0, "the W buffers rotate with the row-block index");
    static_assert(NBUF >= 2 && NBUF <= 4 && 3 * PD <= 63, "vmcnt immediates below");
    __shared__ __attribute__((aligned(1024))) char lds[2 * BUF];
    __shared__ float red_a[kHeadWaves][NB * 16];
    __shared__ float red_b[kHeadWaves][NB * 16];

    const int tid = threadIdx.x;
    const int wave = tid >> 6;
    const int lane = tid & 63;
    const int l16 = lane & 15;
    const int kgp = lane >> 4;
    const int G = gridDim.x;
    const int c = blockIdx.x;
    const int H = p.H, V = p.V;
    const int nch = H / KC;
    const int nsweeps = (p.npasses + NP - 1) / NP;
    const int total_q = nsweeps * nch;
    const int rotc = c % nch;  // workgroups start their K walk at different chunks (HBM channel spread)
    const E sc = (E)p.head_scale;

    // Shared last pass: this workgroup's r_c blocks of it, `share` waves on each (a power of two that
    // divides the chunk count), wave w on block w / share with the chunks q % share == w % share.
    const bool shared_last = p.rem_blocks > 0;
    int r_c = 0, share = 1;
    if (shared_last) {
        r_c = c < p.rem_blocks ? (p.rem_blocks - c + G - 1) / G : 0;
        if (r_c > kHeadWaves) r_c = kHeadWaves;  // cannot happen: rem_blocks <= kHeadWaves * G
        while (r_c > 0 && share * 2 * r_c <= kHeadWaves && nch % (share * 2) == 0) share *= 2;
    }
    const int my_last = wave / share, my_sub = wave % share;
    auto step_active = [&](int q, int pl) -> bool {
        const int pass = (q / nch) * NP + pl;
        if (!shared_last) return pass < p.npasses;
        if (pass != p.full_passes) return pass < p.full_passes;
        return my_last < r_c && (q % share) == my_sub;
    };

    auto chunk_of = [&](int q) { return (q % nch + rotc) % nch; };
    // hidden chunk q -> LDS buffer q & 1 (asynchronous; completion is awaited with vmcnt below)
    auto issue_hidden = [&](int q) {
        const int k0 = chunk_of(q) * KC;
#pragma unroll
        for (int j = 0; j < NINST; ++j) {
            const int inst = wave * NINST + j;
            const int row = inst * (64 / PR) + lane / PR;
            const int piece = (lane % PR) ^ (row & 15);
            const int rc = row < p.n ? row : p.n - 1;  // rows past n: any valid data, their results are dropped
            const f16* src = p.hidden + (size_t)rc * H + k0 + piece * 8;
            const uint32_t dst = __builtin_amdgcn_readfirstlane(
                (uint32_t)(uintptr_t)(__attribute__((address_space(3))) void*)(lds + (q & 1) * BUF + inst * 1024));
            asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(src), "s"(dst) : "memory", "m0");
        }
    };
    auto row_block = [&](int pass) {
        if (shared_last && pass == p.full_passes) return p.full_passes * kHeadWaves * G + c + my_last * G;
        return (pass * kHeadWaves + wave) * G + c;
    };
    int groups_since_dma = 0;  // W groups requested after the newest hidden chunk request
    auto load_w = [&](int q, int pl, X8* buf) {
        const int pass = (q / nch) * NP + pl;
        if (!step_active(q, pl)) return;
        ++groups_since_dma;
        if (p.w_tiled) {  // one contiguous KB per instruction, consecutive steps consecutive in memory
            int rb = row_block(pass);
            rb = rb * 16 < V ? rb : (V - 1) / 16;
            const f16* src = p.w + ((size_t)rb * (H / 32) + chunk_of(q) * (KC / 32)) * 512 + lane * 8;
#pragma unroll
            for (int ks = 0; ks < PD; ++ks) buf[ks] = __builtin_nontemporal_load(reinterpret_cast<const X8*>(src + ks * 512));
            return;
        }
        int row = row_block(pass) * 16 + l16;
        row = row < V ? row : V - 1;  // clamp: rows past the end are computed and discarded
        const f16* src = p.w + (size_t)row * H + chunk_of(q) * KC + kgp * 8;
#pragma unroll
        for (int ks = 0; ks < PD; ++ks) buf[ks] = __builtin_nontemporal_load(reinterpret_cast<const X8*>(src + ks * 32));
    };

    f32x4 acc[NP][NB];
    float ea[NB], eb[NB];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
        ea[nb] = -INFINITY;
        eb[nb] = p.mode == kHeadModeStats ? 0.f : __int_as_float(0x7fffffff);
    }
    const int xl = (kgp ^ (l16 & 3)) << 4, hi = l16 >> 2;

    // W groups are requested NBUF - 1 steps ahead of their use (a step = one row block x one chunk).
    X8 bufs[NBUF][PD];
    issue_hidden(0);
#pragma unroll
    for (int s0 = 0; s0 < NBUF - 1; ++s0) load_w(s0 / NP, s0 % NP, bufs[s0 % NBUF]);  // NBUF - 1 <= NP
    for (int q = 0; q < total_q; ++q) {
        const int ch = q % nch;
        if (ch == 0) {
#pragma unroll
            for (int pl = 0; pl < NP; ++pl)
#pragma unroll
                for (int nb = 0; nb < NB; ++nb)
#pragma unroll
                    for (int r = 0; r < 4; ++r) acc[pl][nb][r] = 0.f;
        }
        // Chunk q was requested one iteration ago.  Memory operations return in order, so it has landed
        // once at most the W groups requested after it -- and never more than the NBUF - 1 that are
        // prefetched ahead -- are still in flight.  (Row blocks past the end request nothing, so the
        // number of groups behind the chunk varies.)
        switch (groups_since_dma < NBUF - 1 ? groups_since_dma : NBUF - 1) {
            case 0: asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); break;
            case 1: asm volatile("s_waitcnt vmcnt(%0)" : : "n"(PD) : "memory"); break;
            case 2: asm volatile("s_waitcnt vmcnt(%0)" : : "n"(2 * PD) : "memory"); break;
            default: asm volatile("s_waitcnt vmcnt(%0)" : : "n"(3 * PD) : "memory"); break;
        }
        if (p.apply_scale) {  // fp16 pre-scale of the hidden rows (src/model/linear.cuh:82-101): own pieces, in place
#pragma unroll
            for (int j = 0; j < NINST; ++j) {
                X8* px = reinterpret_cast<X8*>(lds + (q & 1) * BUF + (wave * NINST + j) * 1024 + lane * 16);
                X8 x = *px;
#pragma unroll
                for (int e = 0; e < 8; ++e) x[e] = (E)((float)x[e] * (float)sc);
                *px = x;
            }
        }
        __syncthreads();  // chunk q visible to all waves; all waves are done with the other buffer
        if (q + 1 < total_q) {
            issue_hidden(q + 1);
            groups_since_dma = 0;
        }
        const char* base = lds + (q & 1) * BUF + l16 * ROWB + xl;
#pragma unroll
        for (int pl = 0; pl < NP; ++pl) {
            {
                constexpr int kA = NBUF - 1;
                const int pn = pl + kA;
                if (pn < NP) load_w(q, pn, bufs[pn % NBUF]);
                else if (q + 1 < total_q) load_w(q + 1, pn - NP, bufs[(pn - NP) % NBUF]);
            }
            if (step_active(q, pl)) {
#pragma unroll
                for (int ks = 0; ks < PD; ++ks) {
                    const char* bk = base + ((ks ^ hi) << 6);
#pragma unroll
                    for (int nb = 0; nb < NB; ++nb) {
                        const X8 b = *reinterpret_cast<const X8*>(bk + nb * 16 * ROWB);
                        acc[pl][nb] = Elem<E>::mfma_16x16x32(bufs[pl % NBUF][ks], b, acc[pl][nb]);
                    }
                }
            }
        }
        if (ch == nch - 1) {
#pragma unroll
            for (int pl = 0; pl < NP; ++pl) {
                const int pass = (q / nch) * NP + pl;
                if (pass < (shared_last ? p.full_passes : p.npasses))
                    head_epilogue<NB, E>(p, acc[pl], row_block(pass) * 16 + kgp * 4, l16, ea, eb);
            }
        }
    }
    if (shared_last) {
        // The waves that shared a block of the last pass hold partial sums over their chunks: they meet in
        // LDS (the hidden buffers are free now) and the first wave of each group adds them up in wave order.
        __syncthreads();
        f32x4* xch = reinterpret_cast<f32x4*>(lds);  // [wave][NB][64 lanes]
        const int pl_last = p.full_passes % NP;
        if (my_last < r_c) {
#pragma unroll
            for (int pl = 0; pl < NP; ++pl)
                if (pl == pl_last)
#pragma unroll
                    for (int nb = 0; nb < NB; ++nb) xch[(wave * NB + nb) * 64 + lane] = acc[pl][nb];
        }
        __syncthreads();
        if (my_last < r_c && my_sub == 0) {
            f32x4 sum[NB];
#pragma unroll
            for (int nb = 0; nb < NB; ++nb) {
                sum[nb] = xch[(wave * NB + nb) * 64 + lane];
                for (int o = 1; o < share; ++o) {
                    const f32x4 x = xch[((wave + o) * NB + nb) * 64 + lane];
#pragma unroll
                    for (int r = 0; r < 4; ++r) sum[nb][r] += x[r];
                }
            }
            head_epilogue<NB, E>(p, sum, row_block(p.full_passes) * 16 + kgp * 4, l16, ea, eb);
        }
    }
    head_finish<NB>(p, ea, eb, red_a, red_b, tid, wave, lane, c);
}

// One finished 16-row block of W in the fused FR-Spec launch: the logits (written through, so that a finisher in another
// XCD can read them once they are marked complete), the running statistics exactly as head_epilogue's STATS branch
// keeps them, and one ranking key per element in LDS: ordered image of z << 16 | (0xFFFF - index within the workgroup).
template <typename E>
__device__ inline void fuse_epilogue(const HeadParams& p, const f32x4& acc, int vrow0, int lidx0, int l16, float& ea, float& eb,
                                     uint32_t* keys_row) {
    if (l16 >= p.n) return;
    typename Elem<E>::x4 zz;
#pragma unroll
    for (int r = 0; r < 4; ++r) zz[r] = (E)acc[r];
    uint32_t kk[4] = {0u, 0u, 0u, 0u};
    if (vrow0 < p.V) {  // V % 8 == 0 in this launch: the four rows are inside or outside together
        fuse_store(reinterpret_cast<uint64_t*>(reinterpret_cast<E*>(p.logits) + (size_t)l16 * p.V + vrow0), __builtin_bit_cast(uint64_t, zz));
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const float x = (float)zz[r];
            kk[r] = (ord16(Elem<E>::to_bits(x)) << 16) | (uint32_t)(0xFFFF - (lidx0 + r));
            if (x == -INFINITY) continue;
            if (x > ea) {
                eb = eb * __expf(ea - x) + 1.f;
                ea = x;
            } else {
                eb += __expf(x - ea);
            }
        }
    }
    *reinterpret_cast<uint4*>(keys_row + lidx0) = make_uint4(kk[0], kk[1], kk[2], kk[3]);
}

// The finisher of hidden row R (all threads of one workgroup, after its own words are out).
template <typename E>
__device__ __forceinline__ void fuse_finish_row(const HeadParams& p, const FuseParams& fp, int R, uint32_t gen_row, uint32_t gen_done) {
    __shared__ uint64_t s_cand[kFuseCap];
    __shared__ uint64_t s_raw[kFuseCap];
    __shared__ uint16_t s_rslice[kFuseCap];
    __shared__ int s_rank[kFuseCap];
    __shared__ uint32_t s_wave_kth[kHeadWaves];
    __shared__ uint64_t s_wave_best[2][kHeadWaves];
    __shared__ float s_m_lse[2];
    __shared__ int s_ncand, s_slow, s_timeout, s_wide;
    HeadFuseState* st = fp.st;
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int G = gridDim.x, top = fp.top, V = p.V;
    const uint32_t g1 = gen_row + 1;
    const uint64_t ctag = (uint64_t)(g1 & kFuseCandTagMask);
    const uint64_t stag = (uint64_t)(g1 & 0xFFFFu);
    // thread -> (workgroup's slice, half of its slots), from the last thread down: wave 0, which reduces the
    // statistics while the others search the bound, is the first to go without data when G < 256
    const int u = kHeadThreads - 1 - tid;
    const int slice = u >> 1, half = u & 1;
    const bool have = slice < G;
    const uint64_t* cw = &st->cand[R][have ? slice : 0][half * 8];
    if (tid == 0) {
        s_ncand = 0;
        s_slow = 0;
        s_timeout = 0;
        s_wide = 0;
    }
    s_cand[tid] = 0;
    s_rank[tid] = 0;
    __syncthreads();
    uint64_t w[8], sw[4];
#pragma unroll
    for (int i = 0; i < 8; ++i) w[i] = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) sw[i] = 0;
    const unsigned long long t_begin = wall_clock64();
    bool late = false;
    for (;;) {
        bool ok = true;
        if (have) {
#pragma unroll
            for (int i = 0; i < 8; ++i) w[i] = fuse_load(cw + i);
#pragma unroll
            for (int i = 0; i < 8; ++i) ok = ok && (w[i] >> 45) == ctag;
        }
        if (wave == 0) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int c = lane + i * 64;
                if (c < G) {
                    sw[i] = fuse_load(&st->stats[R][c]);
                    ok = ok && (sw[i] >> 48) == stag;
                }
            }
        }
        if (ok) break;
        if (wall_clock64() - t_begin >= fp.wait_ticks) {
            late = true;
            break;
        }
        __builtin_amdgcn_s_sleep(1);  // a thread leaves the loop with its own words, so few keep asking towards the end
    }
    if (late) s_timeout = 1;
    __syncthreads();
    CPMCU_STAMP(g_head_timeline, blockIdx.x, 9);
    if (s_timeout) {
        // some workgroup's words never came (it was not resident within the wait): the row is not written; the host
        // reads the count at its next synchronisation and reports the call as failed
        if (tid < top) {
            fp.val[(size_t)R * top + tid] = 0xFFFFu;
            fp.pos[(size_t)R * top + tid] = -1;
            if (fp.ids) fp.ids[(size_t)R * top + tid] = -1;
        }
        if (tid == 0) {
            __hip_atomic_fetch_add(&g_head_fuse_report.timeouts, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            st->gen[R] = g1;
        }
        return;
    }
    uint32_t img[8], tmax = 0, tmin = 0xFFFFFFFFu;
    int nonempty = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        img[i] = (uint32_t)(w[i] >> 29) & 0xFFFFu;
        tmax = img[i] > tmax ? img[i] : tmax;
        if (img[i]) {
            tmin = img[i] < tmin ? img[i] : tmin;
            ++nonempty;
        }
    }
    // k-th largest of this wave's thread maxima (a lower bound of the row's k-th largest value), waves 1..7;
    // wave 0: the row statistics, in the order topk_row_kernel reduces the same partials
    uint32_t kth = 0;
    if (wave != 0) {
        for (int bit = 15; bit >= 4; --bit) {
            const uint32_t c = kth | (1u << bit);
            if (__popcll(__ballot(tmax >= c)) >= top) kth = c;
        }
    } else {
        float pa[4], pb[4];
        bool wide = false;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const bool in = lane + i * 64 < G;
            pa[i] = in ? (float)Elem<E>::from_bits((uint16_t)(sw[i] >> 32)) : -INFINITY;
            pb[i] = in ? __uint_as_float((uint32_t)sw[i] & 0x7FFFFFFFu) : 0.f;
            wide = wide || (in && ((uint32_t)sw[i] >> 31));
        }
        const float a = fmaxf(fmaxf(-INFINITY, fmaxf(pa[0], pa[1])), fmaxf(pa[2], pa[3]));
        float b = 0.f;
#pragma unroll
        for (int i = 0; i < 4; ++i) b += (pa[i] == -INFINITY) ? 0.f : pb[i] * __expf(pa[i] - a);
        const float wm = wave_max_f32(a);
        b = wave_sum_f32((a == -INFINITY) ? 0.f : b * __expf(a - wm));
        const bool any_wide = __ballot(wide) != 0;
        if (lane == 0) {
            const float l = __logf(b);
            s_m_lse[0] = wm;
            s_m_lse[1] = l;
            if (any_wide) s_wide = 1;
            if (fp.row_stats) {
                fp.row_stats[R * 2 + 0] = wm;
                fp.row_stats[R * 2 + 1] = l;
            }
        }
    }
    if (lane == 0) s_wave_kth[wave] = kth;
    __syncthreads();
    CPMCU_STAMP(g_head_timeline, blockIdx.x, 10);
    uint32_t bound = 0;
#pragma unroll
    for (int i = 1; i < kHeadWaves; ++i) bound = s_wave_kth[i] > bound ? s_wave_kth[i] : bound;
    const float m = s_m_lse[0], lse = s_m_lse[1];
    const uint32_t lo = mapped_lower_image<E>(bound, m, lse);
    const auto key_of = [&](uint16_t zbits, int idx) -> uint64_t {
        const float z = Elem<E>::from_bits(zbits);
        return make_key(Elem<E>::to_bits((z - m) - lse), idx);  // src/model/eagle.cuh:87
    };
    {
        // A workgroup published its largest keys only (at least fuse_publish_min of them, or all it had).  What it held
        // back is below all of them, so the candidates of the row are complete unless some workgroup's smallest
        // published value is itself a candidate.
        const uint32_t omin = (uint32_t)__shfl_xor((int)tmin, 1);
        const int ocnt = __shfl_xor(nonempty, 1);
        const uint32_t smin = omin < tmin ? omin : tmin;
        if (lo == 0 || (have && nonempty + ocnt >= fuse_publish_min(top) && smin >= lo)) s_slow = 1;
        // The raw words of everything at or above lo go to LDS: slots by ballot prefix sums, one LDS atomic per wave;
        // the keys are computed afterwards, one candidate per thread.
        const uint64_t lanes_below = (1ull << lane) - 1ull;
        int off[8], total = 0;
        uint32_t em = 0;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const bool is_cand = lo != 0 && img[i] >= lo;
            const uint64_t mk = __ballot(is_cand);
            off[i] = total + __popcll(mk & lanes_below);
            total += __popcll(mk);
            em |= is_cand ? (1u << i) : 0u;
        }
        int base = 0;
        if (lane == 0 && total) base = atomicAdd(&s_ncand, total);
        base = __builtin_amdgcn_readfirstlane(base);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            if ((em & (1u << i)) && base + off[i] < kFuseCap) {
                s_raw[base + off[i]] = w[i];
                s_rslice[base + off[i]] = (uint16_t)slice;
            }
        }
    }
    __syncthreads();
    CPMCU_STAMP(g_head_timeline, blockIdx.x, 11);
    const int C = s_ncand;
    if (!s_slow && C <= kFuseCap) {
        int32_t mapped = 0;
        if (tid < C) {
            const uint64_t x = s_raw[tid];
            const int lidx = (int)((x >> kFuseIdBits) & 0x1FFu);
            const int idx = ((lidx >> 4) * G + (int)s_rslice[tid]) * 16 + (lidx & 15);
            s_cand[tid] = key_of(image_to_bits((uint32_t)(x >> 29) & 0xFFFFu), idx);
            mapped = (int)((uint32_t)x & ((1u << kFuseIdBits) - 1u));
            if (s_wide) mapped = fp.remap ? fp.remap[idx] : idx;
        }
        __syncthreads();
        int shift = 6;
        while ((1 << shift) < C) ++shift;
        const int i = tid & ((1 << shift) - 1);
        const int part = tid >> shift, nparts = kHeadThreads >> shift;
        if (i < C) {
            // slots from C on hold key 0, so whole groups of eight can be compared
            const uint64_t my = s_cand[i];
            const int chunk = ((C + nparts - 1) / nparts + 7) & ~7;
            int r = 0;
            for (int j = part * chunk; j < (part + 1) * chunk && j < kFuseCap; j += 8) {
                uint64_t o[8];
#pragma unroll
                for (int q = 0; q < 8; ++q) o[q] = s_cand[j + q];
#pragma unroll
                for (int q = 0; q < 8; ++q) r += o[q] > my ? 1 : 0;
            }
            if (r) atomicAdd(&s_rank[i], r);
        }
        __syncthreads();
        if (tid < C && s_rank[tid] < top) {
            const uint64_t key = s_cand[tid];
            const size_t o = (size_t)R * top + s_rank[tid];
            fp.val[o] = key_bits(key);
            fp.pos[o] = key_index(key);
            if (fp.ids) fp.ids[o] = mapped;
        }
        CPMCU_STAMP(g_head_timeline, blockIdx.x, 13);
        CPMCU_STAMP_VALUE(g_head_timeline, blockIdx.x, 14, C);
        if (tid == 0) {
            __hip_atomic_fetch_add(&g_head_fuse_report.fused_rows, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            st->gen[R] = g1;
        }
        return;
    }
    // From the logits in memory: every workgroup marks its part complete once its stores have been acknowledged.
    {
        bool late2 = false;
        if (tid < G) {
            while (fuse_load(&st->done[tid]) != (uint64_t)(gen_done + 1)) {
                if (wall_clock64() - t_begin >= fp.wait_ticks) {
                    late2 = true;
                    break;
                }
                __builtin_amdgcn_s_sleep(8);
            }
        }
        if (late2) s_timeout = 1;
    }
    __syncthreads();
    if (s_timeout) {
        if (tid < top) {
            fp.val[(size_t)R * top + tid] = 0xFFFFu;
            fp.pos[(size_t)R * top + tid] = -1;
            if (fp.ids) fp.ids[(size_t)R * top + tid] = -1;
        }
        if (tid == 0) {
            __hip_atomic_fetch_add(&g_head_fuse_report.timeouts, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            st->gen[R] = g1;
        }
        return;
    }
    const uint64_t* xr = reinterpret_cast<const uint64_t*>(reinterpret_cast<const uint16_t*>(p.logits) + (size_t)R * V);
    const int nquads = V >> 2;
    uint64_t prev = ~0ull;
    for (int round = 0; round < top; ++round) {
        uint64_t mine = 0;
        for (int q = tid; q < nquads; q += kHeadThreads) {
            const uint64_t x4 = fuse_load(xr + q);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const uint64_t key = key_of((uint16_t)(x4 >> (16 * e)), q * 4 + e);
                if (key < prev && key > mine) mine = key;
            }
        }
        const uint64_t wbest = wave_max_u64(mine);
        uint64_t* wb = s_wave_best[round & 1];
        if (lane == 0) wb[wave] = wbest;
        __syncthreads();
        uint64_t best = wb[0];
#pragma unroll
        for (int i = 1; i < kHeadWaves; ++i) best = wb[i] > best ? wb[i] : best;
        if (tid == 0 && best != 0) {
            const int idx = key_index(best);
            const size_t o = (size_t)R * top + round;
            fp.val[o] = key_bits(best);
            fp.pos[o] = idx;
            if (fp.ids) fp.ids[o] = fp.remap ? fp.remap[idx] : idx;
        }
        prev = best;
        if (best == 0) break;
    }
    if (tid == 0) {
        __hip_atomic_fetch_add(&g_head_fuse_report.slow_rows, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        st->gen[R] = g1;
    }
}

// Tiled weights whose row blocks fit one sweep: FP full passes (every wave one whole row block each) and at most
// one partly filled last pass.  The wave's W stream is a ring of 1 KB fragments held in registers and refilled
// fragment by fragment: as soon as the MFMAs of a (row block, K step) have read their fragment, the same registers
// are requested again for the same position of the NEXT chunk, so a wave keeps about one chunk's worth of W
// (FP row blocks x KC columns, + its slice of the last pass) in flight at all times.  The loop body is straight-line
// code (FP is a template parameter, the refills are unconditional, the last chunk -- which refills nothing -- is a
// second instance of the body) so that the compiler's own vmcnt bookkeeping is exact: with loads inside
// wave-uniform branches, as in the kernel above, it has to assume the fewest loads in flight, waits for the
// newest group before it computes on the one before, and load and compute take turns.  The scheduling fence
// after every K step keeps the refills where they are written; without it they are sunk below the MFMAs
// that follow, to shorten register live ranges.  Against the kernel above, same GPU, 73448 x 4096 head:
// 103.1 -> 96.2 us with 60 hidden rows, 100.5 -> 95.1 with 33, 92.7 -> 90.3 with 16 or 1.  (Refilling a row
// block's K steps of a chunk in one burst behind its MFMAs instead: 98.7 / 97.4 / 92.0 us.)
//   A K step reads its hidden-row operands from LDS once and uses them for all FP row blocks.
//   Last pass: the workgroup's row blocks of it are shared by `share` waves each (a power of two, the same for
//   the whole launch), and every wave takes `PD / share` K steps of EVERY chunk (slice `wave % share`), so its
//   stream has the same length in every chunk; the partial sums meet in LDS after the loop.  These loads sit in
//   wave-uniform branches (their count is a run-time value); the ring has PD extra slots for them, and what the
//   compiler has to assume about them costs the full passes at most that many fragments of look-ahead.
//   The hidden chunk is brought in as in the kernel above (direct-to-LDS, double buffered, XOR-swizzled).
template <int NB, int FP, int KC, typename E, bool FUSE = false>
__device__ __forceinline__ void head_gemm_stream_body(const HeadParams& p, const FuseParams& fp = FuseParams{}) {
    typedef typename Elem<E>::x8 X8;
    constexpr int PD = KC / 32;              // 1 KB W fragments per row block and chunk
    constexpr int R = (FP + 1) * PD;         // ring slots
    constexpr int ROWB = KC * 2;
    constexpr int BUF = NB * 16 * ROWB;
    constexpr int PR = KC / 8;               // 16-byte pieces per hidden row chunk
    constexpr int NINST = BUF / 1024 / kHeadWaves;  // 1 KB DMA instructions per wave and chunk
    static_assert(NINST >= 1 && PD % 4 == 0 && FP >= 1 && FP * PD <= 63, "shape limits (swizzle groups of 4 K steps, vmcnt immediate)");
    __shared__ __attribute__((aligned(1024))) char lds[2 * BUF];
    __shared__ float red_a[kHeadWaves][NB * 16];
    __shared__ float red_b[kHeadWaves][NB * 16];
    // fused FR-Spec launch: ranking keys [hidden row][element of this workgroup] (row stride padded by one 16-byte
    // piece), token ids of the workgroup's vocabulary rows, the rows' generations, staging of the published slots
    constexpr int kKeyStride = (FP + 1) * 128 + 4;
    __shared__ __attribute__((aligned(16))) uint32_t s_keys[FUSE ? kFuseRows * kKeyStride : 4];
    __shared__ int32_t s_tok[FUSE ? (FP + 1) * 128 : 1];
    __shared__ uint32_t s_gen[kFuseRows];
    __shared__ __attribute__((aligned(16))) uint64_t s_out[FUSE ? kHeadWaves : 1][2 * kFuseSlots];
    __shared__ int s_wave_wide[kHeadWaves];
    __shared__ uint32_t s_ticket;
    static_assert(!FUSE || (NB == 1 && (FP + 1) * 128 <= kHeadThreads), "fused launch: one block of hidden rows, one id per thread");

    const int tid = threadIdx.x;
    const int wave = tid >> 6;
    const int lane = tid & 63;
    const int l16 = lane & 15;
    const int kgp = lane >> 4;
    const int G = gridDim.x;
    const int c = blockIdx.x;
    const int H = p.H;
    const int nch = H / KC;
    const int rotc = c % nch;  // workgroups start their K walk at different chunks (HBM channel spread)
    const E sc = (E)p.head_scale;

    CPMCU_STAMP(g_head_timeline, blockIdx.x, 0);
    int32_t my_tok = 0;
    uint32_t my_gen = 0;
    if constexpr (FUSE) {
        // requested first, so that they return ahead of the W stream: the token id of element `tid` of this workgroup
        // (row block tid / 16 of its blocks, which are G apart) and the generation of hidden row `tid`
        if (tid < (FP + 1) * 128) {
            const int idx = ((tid >> 4) * G + c) * 16 + (tid & 15);
            my_tok = idx < p.V ? (fp.remap ? fp.remap[idx] : idx) : 0;
        }
        if (tid < kFuseRows) my_gen = fp.st->gen[tid];
    }

    // last pass: block `my_last` of this workgroup's share of it, K slice `my_sub` of every chunk
    const int share = p.last_share;
    const int my_last = wave / share, my_sub = wave % share;
    const bool last_active = p.rem_blocks > 0 && c + my_last * G < p.rem_blocks;
    const int sl = last_active ? PD / share : 0;  // K steps per chunk
    const int rb_last = FP * kHeadWaves * G + c + my_last * G;

    auto chunk_of = [&](int q) { const int x = q + rotc; return x >= nch ? x - nch : x; };
    auto issue_hidden = [&](int q) {
        const int k0 = chunk_of(q) * KC;
#pragma unroll
        for (int j = 0; j < NINST; ++j) {
            const int inst = wave * NINST + j;
            const int row = inst * (64 / PR) + lane / PR;
            const int piece = (lane % PR) ^ (row & 15);
            const int rc = row < p.n ? row : p.n - 1;  // rows past n: any valid data, their results are dropped
            const f16* src = p.hidden + (size_t)rc * H + k0 + piece * 8;
            const uint32_t dst = __builtin_amdgcn_readfirstlane(
                (uint32_t)(uintptr_t)(__attribute__((address_space(3))) void*)(lds + (q & 1) * BUF + inst * 1024));
            asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(src), "s"(dst) : "memory", "m0");
        }
    };
    // fragment (row block, 32-column step) of the tiled matrix: 512 halves, this lane's 8 at lane * 8
    const f16* wfull[FP];
#pragma unroll
    for (int pl = 0; pl < FP; ++pl) wfull[pl] = p.w + (size_t)((pl * kHeadWaves + wave) * G + c) * (H / 32) * 512 + lane * 8;
    const f16* wlast = p.w + (size_t)(last_active ? rb_last : 0) * (H / 32) * 512 + lane * 8;
    auto load_frag = [&](const f16* base, int step) { return __builtin_nontemporal_load(reinterpret_cast<const X8*>(base + (size_t)step * 512)); };

    f32x4 acc[FP + 1][NB];
#pragma unroll
    for (int pl = 0; pl <= FP; ++pl)
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[pl][nb][r] = 0.f;
    float ea[NB], eb[NB];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
        ea[nb] = -INFINITY;
        // arg-max: the lane's first vocabulary row stands in until something larger than -inf comes (its rows come in
        // ascending order, so "lowest index among equals" then takes no index comparisons)
        const int first_row = (wave * G + c) * 16 + kgp * 4;
        eb[nb] = p.mode == kHeadModeStats ? 0.f : __int_as_float(first_row < p.V ? first_row : 0x7fffffff);
    }
    const int xl = (kgp ^ (l16 & 3)) << 4, hi = l16 >> 2;

    // ring slot ks * FP + pl: K step ks of full pass pl; slot FP * PD + j: step j of the last-pass slice
    X8 ring[R];
    issue_hidden(0);
    {
        const int s0 = chunk_of(0) * PD;
#pragma unroll
        for (int ks = 0; ks < PD; ++ks)
#pragma unroll
            for (int pl = 0; pl < FP; ++pl) ring[ks * FP + pl] = load_frag(wfull[pl], s0 + ks);
#pragma unroll
        for (int j = 0; j < PD; ++j)
            if (j < sl) ring[FP * PD + j] = load_frag(wlast, s0 + my_sub * sl + j);
    }
    if constexpr (FUSE) {
        for (int i = tid; i < kFuseRows * kKeyStride; i += kHeadThreads) s_keys[i] = 0;
        if (tid < (FP + 1) * 128) s_tok[tid] = my_tok;
        if (tid < kFuseRows) s_gen[tid] = my_gen;
        const bool wide = ((uint32_t)my_tok >> kFuseIdBits) != 0;
        const bool any_wide = __ballot(wide) != 0;
        if (lane == 0) s_wave_wide[wave] = any_wide ? 1 : 0;
    }
    // One chunk: `refill` = request the same ring positions for the next chunk (everywhere but in the last one).
    auto chunk_body = [&](int q, auto refill) {
        // Chunk q of the hidden rows was requested before the FP * PD (+ sl) fragments that were requested since
        // (memory operations return in order).
        asm volatile("s_waitcnt vmcnt(%0)" : : "n"(FP * PD) : "memory");
        if (p.apply_scale) {  // fp16 pre-scale of the hidden rows (src/model/linear.cuh:82-101): own pieces, in place
#pragma unroll
            for (int j = 0; j < NINST; ++j) {
                X8* px = reinterpret_cast<X8*>(lds + (q & 1) * BUF + (wave * NINST + j) * 1024 + lane * 16);
                X8 x = *px;
#pragma unroll
                for (int e = 0; e < 8; ++e) x[e] = (E)((float)x[e] * (float)sc);
                *px = x;
            }
        }
        __syncthreads();  // chunk q visible to all waves; all waves are done with the other buffer
        if (refill) issue_hidden(q + 1);
        const int sn = chunk_of(q + 1) * PD;
        const char* base = lds + (q & 1) * BUF + l16 * ROWB + xl;
        X8 b[2][NB];
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) b[0][nb] = *reinterpret_cast<const X8*>(base + ((0 ^ hi) << 6) + nb * 16 * ROWB);
#pragma unroll
        for (int ks = 0; ks < PD; ++ks) {
            if (ks + 1 < PD) {
#pragma unroll
                for (int nb = 0; nb < NB; ++nb)
                    b[(ks + 1) & 1][nb] = *reinterpret_cast<const X8*>(base + (((ks + 1) ^ hi) << 6) + nb * 16 * ROWB);
            }
#pragma unroll
            for (int pl = 0; pl < FP; ++pl)
#pragma unroll
                for (int nb = 0; nb < NB; ++nb)
                    acc[pl][nb] = Elem<E>::mfma_16x16x32(ring[ks * FP + pl], b[ks & 1][nb], acc[pl][nb]);
            if (refill) {
#pragma unroll
                for (int pl = 0; pl < FP; ++pl) ring[ks * FP + pl] = load_frag(wfull[pl], sn + ks);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int j = 0; j < PD; ++j) {
            if (j < sl) {
                const int ksl = my_sub * sl + j;
                X8 bl[NB];
#pragma unroll
                for (int nb = 0; nb < NB; ++nb) bl[nb] = *reinterpret_cast<const X8*>(base + ((ksl ^ hi) << 6) + nb * 16 * ROWB);
#pragma unroll
                for (int nb = 0; nb < NB; ++nb)
                    acc[FP][nb] = Elem<E>::mfma_16x16x32(ring[FP * PD + j], bl[nb], acc[FP][nb]);
                if (refill) ring[FP * PD + j] = load_frag(wlast, sn + ksl);
            }
        }
    };
    for (int q = 0; q + 1 < nch; ++q) chunk_body(q, std::true_type{});
    chunk_body(nch - 1, std::false_type{});
    CPMCU_STAMP(g_head_timeline, blockIdx.x, 1);
#ifdef CPMCU_TIMELINE
    if (lane == 0 && blockIdx.x < 1024) g_head_timeline[blockIdx.x * 16 + 8 + wave] = wall_clock64();
#endif
    unsigned long long ticket = 0;
    if constexpr (FUSE) {
        // this workgroup's place in the order of finishing (used at the very end; wave 7 has the least to do after the loop)
        if (tid == kHeadThreads - 64) ticket = __hip_atomic_fetch_add(&fp.st->tickets, 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    const auto epilogue = [&](const f32x4 (&a)[NB], int block_pos) {
        if constexpr (FUSE)
            fuse_epilogue<E>(p, a[0], (block_pos * G + c) * 16 + kgp * 4, block_pos * 16 + kgp * 4, l16, ea[0], eb[0], s_keys + l16 * kKeyStride);
        else
            head_epilogue<NB, E, true>(p, a, (block_pos * G + c) * 16 + kgp * 4, l16, ea, eb);
    };
#pragma unroll
    for (int pl = 0; pl < FP; ++pl) epilogue(acc[pl], pl * kHeadWaves + wave);
    CPMCU_STAMP(g_head_timeline, blockIdx.x, 2);
    if (p.rem_blocks > 0) {
        // The waves that shared a block of the last pass hold partial sums over their K slices: they meet in LDS
        // (the hidden buffers are free now) and the first wave of each group adds them up in wave order.
        __syncthreads();
        f32x4* xch = reinterpret_cast<f32x4*>(lds);  // [wave][NB][64 lanes]
        if (last_active && share > 1) {
#pragma unroll
            for (int nb = 0; nb < NB; ++nb) xch[(wave * NB + nb) * 64 + lane] = acc[FP][nb];
        }
        __syncthreads();
        if (FUSE || share == 1) {
            if (last_active && my_sub == 0) {
                for (int o = 1; o < share; ++o) {
#pragma unroll
                    for (int nb = 0; nb < NB; ++nb) {
                        const f32x4 x = xch[((wave + o) * NB + nb) * 64 + lane];
#pragma unroll
                        for (int r = 0; r < 4; ++r) acc[FP][nb][r] += x[r];
                    }
                }
                epilogue(acc[FP], FP * kHeadWaves + my_last);
            }
        } else if (last_active) {
            // every wave of the group takes the blocks of hidden rows nb = my_sub, my_sub + share, ...: the same sums in
            // the same order (slice 0 + slice 1 + ...), a share-th of the additions and of the epilogue each
            const int w0 = wave - my_sub;
#pragma unroll
            for (int nb = 0; nb < NB; ++nb) {
                if ((nb % share) == my_sub) {   // share is a power of two
                    f32x4 x = xch[(w0 * NB + nb) * 64 + lane];
                    for (int o = 1; o < share; ++o) {
                        const f32x4 y = xch[((w0 + o) * NB + nb) * 64 + lane];
#pragma unroll
                        for (int r = 0; r < 4; ++r) x[r] += y[r];
                    }
                    head_epilogue_block<E, true>(p, x, nb, ((FP * kHeadWaves + my_last) * G + c) * 16 + kgp * 4, l16, ea[nb], eb[nb]);
                }
            }
        }
    }
    CPMCU_STAMP(g_head_timeline, blockIdx.x, 3);
    if constexpr (!FUSE) {
        head_finish<NB>(p, ea, eb, red_a, red_b, tid, wave, lane, c);
        CPMCU_STAMP(g_head_timeline, blockIdx.x, 4);
    } else {
        HeadFuseState* st = fp.st;
        // the workgroup's (max, sum exp) of every hidden row, as one tagged word
        head_finish_with<NB>(p, ea, eb, red_a, red_b, tid, wave, lane, [&](int row, float a, float b) {
            if (row >= p.n) return;
            int wide = 0;
#pragma unroll
            for (int i = 0; i < kHeadWaves; ++i) wide |= s_wave_wide[i];
            const uint64_t word = ((uint64_t)((s_gen[row] + 1) & 0xFFFFu) << 48) | ((uint64_t)Elem<E>::to_bits(a) << 32) |
                                  (uint64_t)(__float_as_uint(b) | (wide ? 0x80000000u : 0u));
            fuse_store(&st->stats[row][c], word);
        });
        CPMCU_STAMP(g_head_timeline, blockIdx.x, 4);
        // (head_finish_with has a barrier in it: every wave's keys are in LDS.)  Two hidden rows per wave, one per half
        // of its lanes: the threshold that leaves between fuse_publish_min(k) and 16 of the workgroup's keys of the
        // row, found from the top bit down (keys are unique, so the search ends at exactly that many at the latest).
        const auto select_rows = [&](auto nkl_tag) {
            constexpr int NKL = decltype(nkl_tag)::value;  // keys per lane
            const int half = lane >> 5, l32 = lane & 31;
            const int row = wave * 2 + half;
            if (wave * 2 >= p.n) return;
            uint32_t kk[NKL];
#pragma unroll
            for (int j = 0; j < NKL; ++j) kk[j] = s_keys[row * kKeyStride + l32 + 32 * j];  // rows from n on hold zeros
            const int need = fuse_publish_min(fp.top);
            uint32_t thr_a = 0, thr_b = 0;
            bool done_a = false, done_b = false;
            {
                int ca = 0, cb = 0;
#pragma unroll
                for (int j = 0; j < NKL; ++j) {
                    const uint64_t mk = __ballot(kk[j] != 0u);
                    ca += __popc((uint32_t)mk);
                    cb += __popc((uint32_t)(mk >> 32));
                }
                if (ca <= kFuseSlots) { thr_a = 1; done_a = true; }
                if (cb <= kFuseSlots) { thr_b = 1; done_b = true; }
            }
            for (int bit = 31; bit >= 0 && !(done_a && done_b); --bit) {
                const uint32_t xa = thr_a | (1u << bit), xb = thr_b | (1u << bit);
                const uint32_t x = half ? xb : xa;
                int ca = 0, cb = 0;
#pragma unroll
                for (int j = 0; j < NKL; ++j) {
                    const uint64_t mk = __ballot(kk[j] >= x);
                    ca += __popc((uint32_t)mk);
                    cb += __popc((uint32_t)(mk >> 32));
                }
                if (!done_a && ca >= need) {
                    thr_a = xa;
                    done_a = ca <= kFuseSlots;
                }
                if (!done_b && cb >= need) {
                    thr_b = xb;
                    done_b = cb <= kFuseSlots;
                }
            }
            const uint32_t thr = half ? thr_b : thr_a;
            const uint64_t tagw = (uint64_t)((s_gen[row & (kFuseRows - 1)] + 1) & kFuseCandTagMask) << 45;
            uint64_t* outw = s_out[wave] + half * kFuseSlots;
            if (l32 < kFuseSlots) outw[l32] = tagw;  // empty slot: image 0
            __builtin_amdgcn_wave_barrier();
            const uint32_t below = (1u << l32) - 1u;
            int base = 0;
#pragma unroll
            for (int j = 0; j < NKL; ++j) {
                const bool emit = kk[j] >= thr;
                const uint64_t mk = __ballot(emit);
                const uint32_t mh = half ? (uint32_t)(mk >> 32) : (uint32_t)mk;
                if (emit) {
                    const int slot = base + __popc(mh & below);
                    const uint32_t lidx = 0xFFFFu - (kk[j] & 0xFFFFu);
                    outw[slot] = tagw | ((uint64_t)(kk[j] >> 16) << 29) | ((uint64_t)lidx << kFuseIdBits) |
                                 (uint64_t)((uint32_t)s_tok[lidx] & ((1u << kFuseIdBits) - 1u));
                }
                base += __popc(mh);
            }
            __builtin_amdgcn_wave_barrier();
            if (l32 < kFuseSlots && row < p.n) fuse_store(&st->cand[row][c][l32], outw[l32]);
        };
        if (p.rem_blocks > 0) select_rows(std::integral_constant<int, (FP + 1) * 4>{});
        else select_rows(std::integral_constant<int, FP * 4>{});
        CPMCU_STAMP(g_head_timeline, blockIdx.x, 5);
        // every store of this workgroup acknowledged (the logits among them), then its mark; the ticket has long returned
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        CPMCU_STAMP(g_head_timeline, blockIdx.x, 6);
        if (tid == kHeadThreads - 64) s_ticket = (uint32_t)(ticket % (unsigned long long)G);
        __syncthreads();
        if (tid == 0) fuse_store(&st->done[c], (uint64_t)(s_gen[0] + 1));
        const int place = (int)s_ticket;
        CPMCU_STAMP(g_head_timeline, blockIdx.x, 7);
        CPMCU_STAMP_VALUE(g_head_timeline, blockIdx.x, 12, place + 1);
        if (place < p.n) fuse_finish_row<E>(p, fp, place, s_gen[place], s_gen[0]);
    }
}

// The kernels proper: fp16 under the names they have in every profile, bf16 beside them.
template <int NB>
__global__ __launch_bounds__(kHeadThreads) void head_gemm_kernel(HeadParams p) { head_gemm_body<NB, f16>(p); }
template <int NB>
__global__ __launch_bounds__(kHeadThreads) void head_gemm_bf16_kernel(HeadParams p) { head_gemm_body<NB, bf16>(p); }
template <int NB, int NP, int KC, int NBUF>
__global__ __launch_bounds__(kHeadThreads) void head_gemm_chunked_kernel(HeadParams p) { head_gemm_chunked_body<NB, NP, KC, NBUF, f16>(p); }
template <int NB, int NP, int KC, int NBUF>
__global__ __launch_bounds__(kHeadThreads) void head_gemm_chunked_bf16_kernel(HeadParams p) { head_gemm_chunked_body<NB, NP, KC, NBUF, bf16>(p); }
template <int NB, int FP, int KC>
__global__ __launch_bounds__(kHeadThreads) void head_gemm_stream_kernel(HeadParams p) { head_gemm_stream_body<NB, FP, KC, f16>(p); }
template <int NB, int FP, int KC>
__global__ __launch_bounds__(kHeadThreads) void head_gemm_stream_bf16_kernel(HeadParams p) { head_gemm_stream_body<NB, FP, KC, bf16>(p); }
// FR-Spec head + log-softmax + top-k + id map-back in one launch (one block of hidden rows).
template <int FP, int KC>
__global__ __launch_bounds__(kHeadThreads) void frspec_head_topk_kernel(HeadParams p, FuseParams fp) { head_gemm_stream_body<1, FP, KC, f16, true>(p, fp); }
template <int FP, int KC>
__global__ __launch_bounds__(kHeadThreads) void frspec_head_topk_bf16_kernel(HeadParams p, FuseParams fp) { head_gemm_stream_body<1, FP, KC, bf16, true>(p, fp); }

// Final arg-max over the per-workgroup partials: one block per hidden row.  Largest value, lowest
// index among equals: one 64-bit key (ordered image of the float, complemented index) per partial,
// reduced per wave on the DPP path and across the four waves through LDS.
__global__ __launch_bounds__(256) void head_argmax_finalize_kernel(const float* part_a, const float* part_b,
                                                                   int G, int stride, int32_t* gt) {
    __shared__ uint64_t wave_key[4];
    const int row = blockIdx.x;
    uint64_t best = 0;
    for (int c = threadIdx.x; c < G; c += 256) {
        const float oa = part_a[(size_t)c * stride + row] + 0.f;  // -0 -> +0: they compare equal
        const uint32_t ob = (uint32_t)__float_as_int(part_b[(size_t)c * stride + row]);
        const uint32_t bits = (uint32_t)__float_as_int(oa);
        const uint32_t image = bits ^ ((bits >> 31) ? 0xFFFFFFFFu : 0x80000000u);
        const uint64_t key = ((uint64_t)image << 32) | (0xFFFFFFFFu - ob);
        best = key > best ? key : best;
    }
    best = wave_max_u64(best);
    if ((threadIdx.x & 63) == 0) wave_key[threadIdx.x >> 6] = best;
    __syncthreads();
    if (threadIdx.x == 0) {
#pragma unroll
        for (int w = 1; w < 4; ++w) best = wave_key[w] > best ? wave_key[w] : best;
        gt[row] = (int32_t)(0xFFFFFFFFu - (uint32_t)best);
    }
}

int g_num_cus = 0;

int num_cus() {
    if (g_num_cus == 0) {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
            n = 256;
        g_num_cus = n;
    }
    return g_num_cus;
}

int pick_nb(int n) { return n <= 16 ? 1 : n <= 32 ? 2 : n <= 64 ? 4 : 8; }

}  // namespace

const char* head_shape_name(HeadShape s) {
    switch (s) {
        case HeadShape::Row1: return "head_gemm_kernel<1>";
        case HeadShape::Row2: return "head_gemm_kernel<2>";
        case HeadShape::Row4: return "head_gemm_kernel<4>";
        case HeadShape::Row8: return "head_gemm_kernel<8>";
        case HeadShape::C_1_2_512_2: return "head_gemm_chunked_kernel<1,2,512,2>";
        case HeadShape::C_1_4_256_2: return "head_gemm_chunked_kernel<1,4,256,2>";
        case HeadShape::C_2_4_256_4: return "head_gemm_chunked_kernel<2,4,256,4>";
        case HeadShape::C_2_4_256_2: return "head_gemm_chunked_kernel<2,4,256,2>";
        case HeadShape::C_4_4_256_4: return "head_gemm_chunked_kernel<4,4,256,4>";
        case HeadShape::C_4_4_256_2: return "head_gemm_chunked_kernel<4,4,256,2>";
        case HeadShape::C_8_4_128_2: return "head_gemm_chunked_kernel<8,4,128,2>";
        case HeadShape::C_2_4_512_2: return "head_gemm_chunked_kernel<2,4,512,2>";
        case HeadShape::C_4_4_128_4: return "head_gemm_chunked_kernel<4,4,128,4>";
        case HeadShape::C_8_2_128_2: return "head_gemm_chunked_kernel<8,2,128,2>";
#define CPMCU_X(nb, fp, kc) \
    case HeadShape::S_##nb##_##fp##_##kc: return "head_gemm_stream_kernel<" #nb "," #fp "," #kc ">";
            CPMCU_HEAD_STREAM_SHAPES(CPMCU_X)
#undef CPMCU_X
    }
    return "?";
}

namespace {

// Kernel shapes chosen by measurement on MI355X (73448 x 4096 and 32768 x 4096 heads).
HeadShape pick_head_shape(int NB, int H, bool w_tiled, int nch, int npasses, int nrb, int G, int* full_passes, int* rem_blocks) {
    if (H % 256 != 0 || (!w_tiled && nch <= 2)) {
        // every wave walks whole rows; hidden rows LDS-resident (<= 16 rows) or chunked per row block.
        // Best for row-major weights with <= 16 rows (1 KB runs per row), and the fallback for odd H.
        return NB == 1 ? HeadShape::Row1 : NB == 2 ? HeadShape::Row2 : NB == 4 ? HeadShape::Row4 : HeadShape::Row8;
    }
    if (w_tiled) {
        // one sweep (all passes fit the accumulator sets) with a partly filled last pass: share it
        // (the option head_share_last_pass = 0 keeps the plain mapping; tests compare the two)
        const int rem = nrb - (npasses - 1) * G * kHeadWaves;
        if (npasses <= 4 && rem < G * kHeadWaves && options().head_share_last_pass) {  // <= NP of every shape below
            *full_passes = npasses - 1;
            *rem_blocks = rem;
        }
        // W register buffers: two when a wave works on several row blocks per chunk (the next block's
        // group is the prefetch; 72 vs 65 % of HBM peak for 60 rows, 81 vs 79 % for 10), four when there
        // is a single pass; the FR-Spec head (32768 rows = one block per wave, up to 16 hidden rows) does best
        // with 512-column chunks in two buffers: 47.4 us with its top-k, against 50.0 (256 x 4) and 52.0 (256 x 2)
        const bool deep = npasses == 1;
        switch (NB) {
            case 1: return deep ? HeadShape::C_1_2_512_2 : HeadShape::C_1_4_256_2;
            case 2: return deep ? HeadShape::C_2_4_256_4 : HeadShape::C_2_4_256_2;
            case 4: return deep ? HeadShape::C_4_4_256_4 : HeadShape::C_4_4_256_2;
            default: return HeadShape::C_8_4_128_2;  // 165 vs 190 us with <8,2,128,2> at 128 rows
        }
    }
    switch (NB) {
        // <= 16 rows whose K range exceeds two LDS buffers (H >= 6144): the row-walking kernel, chunked
        case 1: return HeadShape::Row1;
        case 2: return HeadShape::C_2_4_512_2;
        case 4: return HeadShape::C_4_4_128_4;
        default: return HeadShape::C_8_2_128_2;
    }
}

}  // namespace

namespace {
// The shape of one head GEMM: kernel parameters, kernel shape and grid.
int plan_head_gemm(const void* hidden, const void* w, int w_layout, int n, int V, int H, int apply_scale, float head_scale,
                   int mode, void* logits, float* part_a, float* part_b, HeadParams* p_out, HeadShape* shape_out, int* grid_out) {
    CPMCU_CHECK_ARG(w_layout == CPMCU_W_ROW_MAJOR || w_layout == CPMCU_W_TILED, "lm_head: unknown weight layout %d", w_layout);
    const int NB = pick_nb(n);
    const int kc_max = 2048 / NB;
    const int gk = NB <= 4 ? 512 : 256;
    CPMCU_CHECK_ARG(H >= gk && H % gk == 0, "lm_head: hidden size %d must be a multiple of %d for %d rows", H, gk, n);
    HeadParams p;
    p.hidden = (const f16*)hidden;
    p.w = (const f16*)w;
    p.n = n;
    p.V = V;
    p.H = H;
    p.kc = H < kc_max ? H : kc_max;
    CPMCU_CHECK_ARG(H % p.kc == 0, "lm_head: hidden size %d not divisible by the K chunk %d", H, p.kc);
    p.nch = H / p.kc;
    p.apply_scale = apply_scale;
    p.head_scale = head_scale;
    p.mode = mode;
    p.w_tiled = w_layout == CPMCU_W_TILED;
    p.logits = (f16*)logits;
    p.part_a = part_a;
    p.part_b = part_b;
    const int nrb = ceil_div(V, 16);
    int G = num_cus();
    if (G * kHeadWaves > nrb) G = ceil_div(nrb, kHeadWaves);
    // The streaming kernel has accumulators for four full passes per wave (two for 65 to 128 hidden rows: three or four
    // spill), so a vocabulary of more passes than that gets a multiple of the CU count in workgroups -- they run one after
    // the other on a CU, the stream does not stop between them -- instead of the K-chunked kernel (128 rows x 151936 x 4096:
    // 0.75 against 0.53 of HBM peak; 60 rows x 200000 x 4096: 0.82 against 0.76; 1 to 60 rows x 262144 x 4096: 0.81 against
    // 0.81 to 0.83).
    const int stream_passes = NB == 8 ? 2 : 4;
    if (p.w_tiled && options().head_stream_kernel && H % (NB == 8 ? 128 : 256) == 0 && nrb / (G * kHeadWaves) > stream_passes) {
        const int m = nrb / (G * kHeadWaves * (stream_passes + 1)) + 1;
        if (G * m <= head_max_grid()) G *= m;
    }
    p.npasses = ceil_div(nrb, G * kHeadWaves);
    p.full_passes = 0;
    p.rem_blocks = 0;
    CPMCU_CHECK_ARG(G <= head_max_grid(), "lm_head: %d workgroups exceed the %d rows of the partial planes", G, head_max_grid());
    *grid_out = G;
    p.last_share = 1;
    HeadShape shape = pick_head_shape(NB, H, p.w_tiled, p.nch, p.npasses, nrb, G, &p.full_passes, &p.rem_blocks);
    // Tiled weights with 1..4 full passes (1..2 for 65-128 hidden rows) and at most one partly filled pass: the streaming kernel.
    int stream_kc = 0;
    if (p.w_tiled && options().head_stream_kernel) {
        const int slots = G * kHeadWaves;
        const int full = nrb / slots, rem = nrb % slots;
#define CPMCU_X(nb, fp, kc)                                \
    if (NB == nb && full == fp && H % kc == 0) {           \
        shape = HeadShape::S_##nb##_##fp##_##kc;           \
        stream_kc = kc;                                    \
    }
        CPMCU_HEAD_STREAM_SHAPES(CPMCU_X)
#undef CPMCU_X
        if (stream_kc) {
            p.full_passes = full;
            p.rem_blocks = rem;
            if (rem > 0 && options().head_share_last_pass) {
                // the busiest workgroup has r_max blocks of the last pass; share * r_max waves work on them
                const int r_max = ceil_div(rem, G);
                while (p.last_share * 2 * r_max <= kHeadWaves && p.last_share * 2 <= stream_kc / 32) p.last_share *= 2;
            }
        }
    }
    *shape_out = shape;
    *p_out = p;
    return CPMCU_OK;
}
}  // namespace

// Shared launcher of the GEMM; returns the grid size used (= number of partial rows) in *grid_out.
int launch_head_gemm(const void* hidden, const void* w, int w_layout, int n, int V, int H, int apply_scale, float head_scale,
                     int mode, void* logits, float* part_a, float* part_b, int* grid_out, int* stride_out,
                     hipStream_t st, HeadShape* shape_out, bool dry_run) {
    HeadParams p;
    HeadShape shape;
    int G = 0;
    const int rc = plan_head_gemm(hidden, w, w_layout, n, V, H, apply_scale, head_scale, mode, logits, part_a, part_b, &p, &shape, &G);
    if (rc != CPMCU_OK) return rc;
    *grid_out = G;
    *stride_out = pick_nb(n) * 16;
    if (shape_out) *shape_out = shape;
    if (dry_run) return CPMCU_OK;
    const bool is_bf16 = options().dtype == 1;
#define CPMCU_HEAD_ROW(nb)                                                                                   \
    do {                                                                                                     \
        if (is_bf16) hipLaunchKernelGGL(head_gemm_bf16_kernel<nb>, dim3(G), dim3(kHeadThreads), 0, st, p);    \
        else hipLaunchKernelGGL(head_gemm_kernel<nb>, dim3(G), dim3(kHeadThreads), 0, st, p);                 \
    } while (0)
#define CPMCU_HEAD_CHUNKED(nb, np, kc, nbuf)                                                                                     \
    do {                                                                                                                         \
        if (is_bf16) hipLaunchKernelGGL((head_gemm_chunked_bf16_kernel<nb, np, kc, nbuf>), dim3(G), dim3(kHeadThreads), 0, st, p); \
        else hipLaunchKernelGGL((head_gemm_chunked_kernel<nb, np, kc, nbuf>), dim3(G), dim3(kHeadThreads), 0, st, p);              \
    } while (0)
    switch (shape) {
        case HeadShape::Row1: CPMCU_HEAD_ROW(1); break;
        case HeadShape::Row2: CPMCU_HEAD_ROW(2); break;
        case HeadShape::Row4: CPMCU_HEAD_ROW(4); break;
        case HeadShape::Row8: CPMCU_HEAD_ROW(8); break;
        case HeadShape::C_1_2_512_2: CPMCU_HEAD_CHUNKED(1, 2, 512, 2); break;
        case HeadShape::C_1_4_256_2: CPMCU_HEAD_CHUNKED(1, 4, 256, 2); break;
        case HeadShape::C_2_4_256_4: CPMCU_HEAD_CHUNKED(2, 4, 256, 4); break;
        case HeadShape::C_2_4_256_2: CPMCU_HEAD_CHUNKED(2, 4, 256, 2); break;
        case HeadShape::C_4_4_256_4: CPMCU_HEAD_CHUNKED(4, 4, 256, 4); break;
        case HeadShape::C_4_4_256_2: CPMCU_HEAD_CHUNKED(4, 4, 256, 2); break;
        case HeadShape::C_8_4_128_2: CPMCU_HEAD_CHUNKED(8, 4, 128, 2); break;
        case HeadShape::C_2_4_512_2: CPMCU_HEAD_CHUNKED(2, 4, 512, 2); break;
        case HeadShape::C_4_4_128_4: CPMCU_HEAD_CHUNKED(4, 4, 128, 4); break;
        case HeadShape::C_8_2_128_2: CPMCU_HEAD_CHUNKED(8, 2, 128, 2); break;
#define CPMCU_X(nb, fp, kc)                                                                                                   \
    case HeadShape::S_##nb##_##fp##_##kc:                                                                                     \
        if (is_bf16) hipLaunchKernelGGL((head_gemm_stream_bf16_kernel<nb, fp, kc>), dim3(G), dim3(kHeadThreads), 0, st, p);   \
        else hipLaunchKernelGGL((head_gemm_stream_kernel<nb, fp, kc>), dim3(G), dim3(kHeadThreads), 0, st, p);                \
        break;
            CPMCU_HEAD_STREAM_SHAPES(CPMCU_X)
#undef CPMCU_X
    }
#undef CPMCU_HEAD_ROW
#undef CPMCU_HEAD_CHUNKED
    CPMCU_LAUNCH_CHECK();
    return CPMCU_OK;
}

int head_max_grid() { return 1024; }

// ---- host side of the fused FR-Spec launch -----------------------------------------------------------------------
namespace {
constexpr int kFuseDevices = 64;
std::mutex g_fuse_mu;
struct FuseKey {
    int dev;
    const void* workspace;
    int grid;
    bool operator<(const FuseKey& o) const { return std::tie(dev, workspace, grid) < std::tie(o.dev, o.workspace, o.grid); }
};
std::map<FuseKey, int> g_fuse_states;         // -> index into the device's g_head_fuse
std::vector<int> g_fuse_free[kFuseDevices];
bool g_fuse_listed[kFuseDevices] = {false};
bool g_fuse_off[kFuseDevices] = {false};      // a finisher's wait ran out on this device: back to two launches
HeadFuseState* g_fuse_base[kFuseDevices] = {nullptr};
HeadFuseReport* g_fuse_report_host[kFuseDevices] = {nullptr};

// The state a (workspace, grid) pair publishes its words through, on the current device; null: none left, or the
// first use on the device falls inside a stream capture (the address lookup does not belong there).  States stay with
// their pair until the workspace is released: launches that were captured into a graph keep using them.
HeadFuseState* fuse_state_for(const void* workspace, int grid, hipStream_t st, bool create) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kFuseDevices) return nullptr;
    std::lock_guard<std::mutex> lock(g_fuse_mu);
    if (g_fuse_off[dev]) return nullptr;
    auto it = g_fuse_states.find({dev, workspace, grid});
    if (it == g_fuse_states.end()) {
        if (!create) return nullptr;
        if (g_fuse_base[dev] == nullptr) {
            hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
            if (hipStreamIsCapturing(st, &capturing) != hipSuccess || capturing != hipStreamCaptureStatusNone) {
                (void)hipGetLastError();
                return nullptr;
            }
            void* ptr = nullptr;
            if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(g_head_fuse)) != hipSuccess) {
                (void)hipGetLastError();
                return nullptr;
            }
            g_fuse_base[dev] = (HeadFuseState*)ptr;
        }
        if (!g_fuse_listed[dev]) {
            for (int b = kFuseStates - 1; b >= 0; --b) g_fuse_free[dev].push_back(b);
            g_fuse_listed[dev] = true;
        }
        if (g_fuse_free[dev].empty()) return nullptr;
        const int b = g_fuse_free[dev].back();
        g_fuse_free[dev].pop_back();
        it = g_fuse_states.emplace(FuseKey{dev, workspace, grid}, b).first;
    }
    return g_fuse_base[dev] + it->second;
}

// Whether this call takes the one-launch form, and with which kernel.
bool fuse_eligible(const HeadParams& p, HeadShape shape, int G, int k, const void* logits) {
    if (!options().frspec_fused || !options().head_stream_kernel) return false;
    if (shape != HeadShape::S_1_1_512 && shape != HeadShape::S_1_2_256) return false;
    return G >= kFuseRows && G <= kFuseMaxGrid && p.n <= kFuseRows && k <= kFuseSlots && p.V % 8 == 0 && p.V <= (1 << kFuseIdBits) &&
           ((uintptr_t)logits & 7) == 0;
}
}  // namespace

// FR-Spec head + log-softmax + top-k + id map-back as one launch when the shape allows it (tiled weights, <= 16 hidden
// rows, k <= 16, one or two full passes of row blocks) and a state is to be had; *launched says whether it was.
int launch_frspec_fused(const void* hidden, const void* w, int w_layout, const int32_t* token_id_remap, int n, int V, int H, int k,
                        void* logits, float* row_stats, void* topk_val, int32_t* topk_pos, int32_t* topk_ids, const void* workspace,
                        hipStream_t st, bool* launched, bool dry_run) {
    *launched = false;
    if (w_layout != CPMCU_W_TILED || n > kFuseRows) return CPMCU_OK;
    HeadParams p;
    HeadShape shape;
    int G = 0;
    const int rc = plan_head_gemm(hidden, w, w_layout, n, V, H, 0, 1.f, kHeadModeStats, logits, nullptr, nullptr, &p, &shape, &G);
    if (rc != CPMCU_OK) return rc;
    if (!fuse_eligible(p, shape, G, k, logits)) return CPMCU_OK;
    HeadFuseState* state = fuse_state_for(workspace, G, st, true);
    if (state == nullptr) return CPMCU_OK;
    *launched = true;
    if (dry_run) return CPMCU_OK;
    FuseParams fp;
    fp.st = state;
    fp.top = k;
    fp.remap = token_id_remap;
    fp.val = (uint16_t*)topk_val;
    fp.pos = topk_pos;
    fp.ids = topk_ids;
    fp.row_stats = row_stats;
    fp.wait_ticks = (uint32_t)options().frspec_wait_us * 100u;
    const bool is_bf16 = options().dtype == 1;
    if (shape == HeadShape::S_1_1_512) {
        if (is_bf16) hipLaunchKernelGGL((frspec_head_topk_bf16_kernel<1, 512>), dim3(G), dim3(kHeadThreads), 0, st, p, fp);
        else hipLaunchKernelGGL((frspec_head_topk_kernel<1, 512>), dim3(G), dim3(kHeadThreads), 0, st, p, fp);
    } else {
        if (is_bf16) hipLaunchKernelGGL((frspec_head_topk_bf16_kernel<2, 256>), dim3(G), dim3(kHeadThreads), 0, st, p, fp);
        else hipLaunchKernelGGL((frspec_head_topk_kernel<2, 256>), dim3(G), dim3(kHeadThreads), 0, st, p, fp);
    }
    CPMCU_LAUNCH_CHECK();
    return CPMCU_OK;
}

// Gives back the states of a workspace that is about to be freed (none of its launches in flight or captured).
void head_fuse_release_workspace(const void* workspace) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kFuseDevices) return;
    std::lock_guard<std::mutex> lock(g_fuse_mu);
    for (auto it = g_fuse_states.begin(); it != g_fuse_states.end();) {
        if (it->first.dev == dev && it->first.workspace == workspace) {
            g_fuse_free[dev].push_back(it->second);
            it = g_fuse_states.erase(it);
        } else {
            ++it;
        }
    }
}

// The report words of the current device, copied to pinned host memory in stream order (ahead of a synchronisation,
// never under a capture) and looked at afterwards; a wait that ran out switches the device back to two launches.
int head_fuse_report_enqueue(hipStream_t st) {
    int dev = 0;
    CPMCU_HIP(hipGetDevice(&dev));
    CPMCU_CHECK_ARG(dev >= 0 && dev < kFuseDevices, "device index %d outside [0, %d)", dev, kFuseDevices);
    if (g_fuse_report_host[dev] == nullptr) {
        CPMCU_HIP(hipHostMalloc((void**)&g_fuse_report_host[dev], sizeof(HeadFuseReport), hipHostMallocDefault));
        *g_fuse_report_host[dev] = HeadFuseReport{0u, 0u, 0u};
    }
    CPMCU_HIP(hipMemcpyFromSymbolAsync(g_fuse_report_host[dev], HIP_SYMBOL(g_head_fuse_report), sizeof(HeadFuseReport), 0, hipMemcpyDeviceToHost, st));
    return CPMCU_OK;
}
int head_fuse_report_take(unsigned int* timeouts, unsigned int* slow_rows, unsigned int* fused_rows) {
    int dev = 0;
    CPMCU_HIP(hipGetDevice(&dev));
    *timeouts = *slow_rows = *fused_rows = 0;
    if (dev < 0 || dev >= kFuseDevices || g_fuse_report_host[dev] == nullptr) return CPMCU_OK;
    const HeadFuseReport r = *g_fuse_report_host[dev];
    if (r.timeouts != 0 || r.slow_rows != 0 || r.fused_rows != 0) {
        const HeadFuseReport zero{0u, 0u, 0u};
        CPMCU_HIP(hipMemcpyToSymbol(HIP_SYMBOL(g_head_fuse_report), &zero, sizeof(zero)));
        *g_fuse_report_host[dev] = zero;
        if (r.timeouts != 0) {
            std::lock_guard<std::mutex> lock(g_fuse_mu);
            g_fuse_off[dev] = true;
        }
    }
    *timeouts = r.timeouts;
    *slow_rows = r.slow_rows;
    *fused_rows = r.fused_rows;
    return CPMCU_OK;
}
void head_fuse_reenable() {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kFuseDevices) return;
    std::lock_guard<std::mutex> lock(g_fuse_mu);
    g_fuse_off[dev] = false;
}

}  // namespace cpmcu

using namespace cpmcu;

extern "C" size_t cpmcu_head_workspace_bytes(int n, int V) {
    if (n <= 0 || V <= 0) return 0;
    // per-workgroup partials (two float planes) + top-k candidates (see topk.hip)
    const size_t parts = (size_t)2 * head_max_grid() * 128 * sizeof(float);
    return align_up(parts, 256) + cpmcu_topk_workspace_bytes(n, V, 32);
}

// Re-tiles a [V][H] row-major weight matrix (optionally gathering rows through `row_remap`, which fuses
// remap_copy, src/model/tree_drafter.cuh:79-86) into MFMA operand order: one workgroup per 16-row block.
__global__ __launch_bounds__(256) void head_weight_tile_kernel(const f16x8* __restrict__ w, const int32_t* __restrict__ row_remap, int V,
                                                               int H, f16x8* __restrict__ out) {
    const int rb = blockIdx.x;
    const int steps = H / 32;
    for (int x = threadIdx.x; x < steps * 64; x += 256) {
        const int ks = x >> 6, lane = x & 63;
        const int row = rb * 16 + (lane & 15);
        f16x8 v;
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = (f16)0.f;
        if (row < V) {
            const size_t src_row = row_remap ? (size_t)row_remap[row] : (size_t)row;
            v = w[(src_row * H + ks * 32 + (lane >> 4) * 8) / 8];
        }
        out[((size_t)rb * steps + ks) * 64 + lane] = v;
    }
}

extern "C" size_t cpmcu_head_weight_tiled_bytes(int V, int H) {
    if (V <= 0 || H <= 0) return 0;
    return (size_t)ceil_div(V, 16) * 16 * H * sizeof(f16);
}

extern "C" int cpmcu_head_weight_tile(const void* w, const int32_t* row_remap, int V, int H, void* w_tiled, void* stream) {
    CPMCU_CHECK_ARG(w && w_tiled && w != w_tiled, "head_weight_tile: null or aliased pointer argument");
    CPMCU_CHECK_ARG(V >= 1 && H >= 32 && H % 32 == 0, "head_weight_tile: V=%d, H=%d must be a positive multiple of 32", V, H);
    hipLaunchKernelGGL(head_weight_tile_kernel, dim3(ceil_div(V, 16)), dim3(256), 0, resolve_stream(stream), (const f16x8*)w, row_remap, V, H,
                       (f16x8*)w_tiled);
    CPMCU_LAUNCH_CHECK();
    return CPMCU_OK;
}

// The target head on per-workgroup partials held at `part_a` (two float planes of head_max_grid() * 128).
static int lm_head_argmax_on(const void* hidden, const void* w, int w_layout, int n, int V, int H, int apply_scale,
                             float head_scale, void* logits, int32_t* gt, float* part_a, hipStream_t st) {
    float* part_b = part_a + (size_t)head_max_grid() * 128;
    int G = 0, stride = 0;
    int rc = launch_head_gemm(hidden, w, w_layout, n, V, H, apply_scale, head_scale, kHeadModeArgmax, logits, part_a, part_b, &G, &stride, st, nullptr, false);
    if (rc != CPMCU_OK) return rc;
    if (gt) {
        hipLaunchKernelGGL(head_argmax_finalize_kernel, dim3(n), dim3(256), 0, st, part_a, part_b, G, stride, gt);
        CPMCU_LAUNCH_CHECK();
    }
    return CPMCU_OK;
}

extern "C" int cpmcu_lm_head_argmax(const void* hidden, const void* w, int w_layout, int n, int V, int H, int apply_scale,
                                    float head_scale, void* logits, int32_t* gt, void* workspace,
                                    size_t workspace_bytes, void* stream) {
    CPMCU_CHECK_ARG(hidden && w, "lm_head_argmax: null pointer argument");
    CPMCU_CHECK_ARG(n >= 1 && n <= 128, "lm_head_argmax: n=%d outside [1, 128]", n);
    CPMCU_CHECK_ARG(V >= 1 && H >= 1, "lm_head_argmax: bad shape V=%d H=%d", V, H);
    CPMCU_CHECK_ARG(logits || gt, "lm_head_argmax: both outputs are null");
    CPMCU_CHECK_ARG(workspace && workspace_bytes >= cpmcu_head_workspace_bytes(n, V),
                    "lm_head_argmax: workspace of %zu bytes needed, %zu given", cpmcu_head_workspace_bytes(n, V), workspace_bytes);
    return lm_head_argmax_on(hidden, w, w_layout, n, V, H, apply_scale, head_scale, logits, gt, (float*)workspace, resolve_stream(stream));
}

// Which kernel a head call of this shape launches (no launch): the name for reports.
extern "C" int cpmcu_head_plan(int n, int V, int H, int w_layout, char* kernel_name, size_t kernel_name_bytes, int* num_workgroups) {
    CPMCU_CHECK_ARG(n >= 1 && n <= 128 && V >= 1 && H >= 1, "head_plan: bad shape n=%d V=%d H=%d", n, V, H);
    HeadShape shape;
    int G = 0, stride = 0;
    int rc = launch_head_gemm(nullptr, nullptr, w_layout, n, V, H, 0, 1.f, kHeadModeArgmax, nullptr, nullptr, nullptr, &G, &stride, nullptr,
                              &shape, true);
    if (rc != CPMCU_OK) return rc;
    if (kernel_name && kernel_name_bytes > 0) snprintf(kernel_name, kernel_name_bytes, "%s", head_shape_name(shape));
    if (num_workgroups) *num_workgroups = G;
    return CPMCU_OK;
}

// The GEMM alone: the arg-max stays in per-workgroup partials for cpmcu_verify_tail to finish.
extern "C" int cpmcu_lm_head_partials(const void* hidden, const void* w, int w_layout, int n, int V, int H, int apply_scale,
                                      float head_scale, void* logits, void* workspace, size_t workspace_bytes, int* num_partials,
                                      int* partial_stride, void* stream) {
    CPMCU_CHECK_ARG(hidden && w && num_partials && partial_stride, "lm_head_partials: null pointer argument");
    CPMCU_CHECK_ARG(n >= 1 && n <= 128, "lm_head_partials: n=%d outside [1, 128]", n);
    CPMCU_CHECK_ARG(V >= 1 && H >= 1, "lm_head_partials: bad shape V=%d H=%d", V, H);
    CPMCU_CHECK_ARG(workspace && workspace_bytes >= cpmcu_head_workspace_bytes(n, V),
                    "lm_head_partials: workspace of %zu bytes needed, %zu given", cpmcu_head_workspace_bytes(n, V), workspace_bytes);
    float* part_a = (float*)workspace;
    float* part_b = part_a + (size_t)head_max_grid() * 128;
    return launch_head_gemm(hidden, w, w_layout, n, V, H, apply_scale, head_scale, kHeadModeArgmax, logits, part_a, part_b, num_partials,
                            partial_stride, resolve_stream(stream), nullptr, false);
}

// ---- the same operator for callers that cannot allocate ----
// The per-workgroup partials live in a file-scope device array instead of a caller-provided workspace.
// Every GPU holds its own copy of the array at its own address; the address is looked up once per
// device (with that device current) and kept.  On the host the array's name is only a handle for that
// lookup -- kernels are always given the looked-up pointer.
namespace {
constexpr int kStaticHeadMaxRows = 128;
constexpr size_t kStaticHeadScratchBytes = (size_t)2 * 1024 * kStaticHeadMaxRows * sizeof(float);  // both partial planes: 1 MiB
static __device__ __align__(256) unsigned char scratch[kStaticHeadScratchBytes];
constexpr int kMaxDevices = 64;
void* g_scratch_ptr[kMaxDevices] = {};
std::mutex g_scratch_mutex;

int static_head_scratch(float** out, hipStream_t st) {
    int dev = -1;
    CPMCU_HIP(hipGetDevice(&dev));
    CPMCU_CHECK_ARG(dev >= 0 && dev < kMaxDevices, "lm_head_argmax_static: device index %d outside [0, %d)", dev, kMaxDevices);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (g_scratch_ptr[dev] == nullptr) {
        // The address lookup is not a thing to do while the stream is being captured: the first call on a device has to
        // come before.
        hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing(st, &capturing) != hipSuccess) (void)hipGetLastError();
        CPMCU_CHECK_ARG(capturing == hipStreamCaptureStatusNone,
                        "lm_head_argmax_static: the first call on a device looks up the address of the built-in scratch and cannot be "
                        "part of a stream capture; make one call outside the capture first");
        void* ptr = nullptr;
        CPMCU_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
        g_scratch_ptr[dev] = ptr;
    }
    *out = (float*)g_scratch_ptr[dev];
    return CPMCU_OK;
}
}  // namespace

extern "C" size_t cpmcu_lm_head_argmax_static_scratch_bytes(void) { return kStaticHeadScratchBytes; }

extern "C" int cpmcu_lm_head_argmax_static(const void* hidden, const void* w, int w_layout, int n, int V, int H, int apply_scale,
                                           float head_scale, void* logits, int32_t* gt, void* stream) {
    CPMCU_CHECK_ARG(hidden && w, "lm_head_argmax_static: null pointer argument");
    CPMCU_CHECK_ARG(n >= 1 && n <= kStaticHeadMaxRows, "lm_head_argmax_static: n=%d outside [1, %d], the rows the built-in scratch holds",
                    n, kStaticHeadMaxRows);
    CPMCU_CHECK_ARG(V >= 1 && H >= 1, "lm_head_argmax_static: bad shape V=%d H=%d", V, H);
    CPMCU_CHECK_ARG(logits || gt, "lm_head_argmax_static: both outputs are null");
    static_assert(kStaticHeadScratchBytes >= (size_t)2 * 1024 * 128 * sizeof(float), "two planes of head_max_grid() x 128 floats");
    CPMCU_CHECK_ARG(head_max_grid() * 128 * 2 * sizeof(float) <= kStaticHeadScratchBytes,
                    "lm_head_argmax_static: the built-in scratch of %zu bytes is too small for %d workgroups", kStaticHeadScratchBytes,
                    head_max_grid());
    float* part = nullptr;
    int rc = static_head_scratch(&part, (hipStream_t)stream);
    if (rc != CPMCU_OK) return rc;
    // NULL selects HIP's null stream here: the library's own stream is created on first use, and this entry
    // point creates nothing
    return lm_head_argmax_on(hidden, w, w_layout, n, V, H, apply_scale, head_scale, logits, gt, part, (hipStream_t)stream);
}

CPMCU_TIMELINE_READER(cpmcu_timeline_read_head, cpmcu::g_head_timeline)
