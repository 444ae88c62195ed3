// CPU oracle -- TEST INFRASTRUCTURE ONLY (see cpmcu_oracle.h for the contract,
// the reference citations of every function and what pins each of them).
//
// Build: make -C oracle   (g++ -O3 -march=x86-64-v3 -fopenmp, no GPU deps)

#include "cpmcu_oracle.h"

#include <algorithm>
#include <cmath>
#include <cstring>
#include <limits>
#include <numeric>
#include <vector>

#ifdef _OPENMP
#include <omp.h>
#endif
#ifdef __F16C__
#include <immintrin.h>
#endif

namespace {

int g_threads = 0;  // 0 = OpenMP default

// ---- software binary16 <-> binary32 (reference implementation; the F16C
// path below must agree with it bit for bit, which the unit tests check) ----
inline float half_to_float_sw(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1Fu;
    uint32_t man = h & 0x3FFu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else {  // subnormal: normalise
            int e = -1;
            do { man <<= 1; ++e; } while ((man & 0x400u) == 0);
            bits = sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3FFu) << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7F800000u | (man << 13);
    } else {
        bits = sign | ((exp + 112u) << 23) | (man << 13);
    }
    float f;
    std::memcpy(&f, &bits, 4);
    return f;
}

inline uint16_t float_to_half_sw(float f) {
    uint32_t x;
    std::memcpy(&x, &f, 4);
    uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
    uint32_t absx = x & 0x7FFFFFFFu;
    if (absx >= 0x7F800000u) {  // inf / nan
        return (uint16_t)(sign | 0x7C00u | (absx > 0x7F800000u ? 0x200u | ((absx >> 13) & 0x3FFu) : 0u));
    }
    if (absx >= 0x477FF000u) {  // >= 65520 rounds to inf
        return (uint16_t)(sign | 0x7C00u);
    }
    if (absx < 0x33000001u) {  // <= 2^-25 rounds to zero (tie at exactly 2^-25 -> even = 0)
        return sign;
    }
    int32_t e = (int32_t)(absx >> 23) - 127;
    uint32_t m = (absx & 0x7FFFFFu) | 0x800000u;
    int shift;
    uint32_t base;
    if (e < -14) {  // subnormal half: value = m * 2^(e-23), unit = 2^-24
        shift = 13 + (-14 - e);
        base = 0;
    } else {
        shift = 13;
        base = ((uint32_t)(e + 15) << 10) - 0x400u;  // hidden bit of m adds 0x400
    }
    uint32_t q = m >> shift;
    uint32_t rem = m & ((1u << shift) - 1u);
    uint32_t half = 1u << (shift - 1);
    if (rem > half || (rem == half && (q & 1u))) ++q;
    return (uint16_t)(sign | (base + q));
}

// ---- bfloat16 <-> binary32: the upper half of the binary32 pattern, round to nearest even; a NaN stays a (quiet) NaN ----
inline float bf16_to_float(uint16_t h) {
    const uint32_t bits = (uint32_t)h << 16;
    float f;
    std::memcpy(&f, &bits, 4);
    return f;
}
inline uint16_t float_to_bf16(float f) {
    uint32_t x;
    std::memcpy(&x, &f, 4);
    if ((x & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((x >> 16) | 0x0040u);
    x += 0x7FFFu + ((x >> 16) & 1u);
    return (uint16_t)(x >> 16);
}

// The 16-bit element type of every tensor that crosses the interface: 0 = IEEE binary16 (the default), 1 = bfloat16
// (src/entry.cu:26-59 dispatches the reference's templates on the same two).  Set once, ahead of the calls it governs.
int g_dtype = 0;

inline float half_to_float(uint16_t h) {
#ifdef __F16C__
    return _cvtsh_ss(h);
#else
    return half_to_float_sw(h);
#endif
}
inline uint16_t float_to_half(float f) {
#ifdef __F16C__
    return _cvtss_sh(f, _MM_FROUND_TO_NEAREST_INT | _MM_FROUND_NO_EXC);
#else
    return float_to_half_sw(f);
#endif
}
// the element type in force
inline float h2f(uint16_t h) { return g_dtype == 1 ? bf16_to_float(h) : half_to_float(h); }
inline uint16_t f2h(float f) { return g_dtype == 1 ? float_to_bf16(f) : float_to_half(f); }

// dot product with 16 interleaved fp32 partial sums (lane = k mod 16) and a
// fixed pairwise tree at the end.  n must be a multiple of 16.
inline float dot16(const float* a, const float* b, int n) {
    float acc[16];
    for (int j = 0; j < 16; ++j) acc[j] = 0.f;
    for (int k = 0; k < n; k += 16) {
        for (int j = 0; j < 16; ++j) acc[j] = std::fma(a[k + j], b[k + j], acc[j]);
    }
    for (int w = 8; w >= 1; w >>= 1)
        for (int j = 0; j < w; ++j) acc[j] += acc[j + w];
    return acc[0];
}

inline float dot_any(const float* a, const float* b, int n) {
    int n16 = n & ~15;
    float r = n16 ? dot16(a, b, n16) : 0.f;
    for (int k = n16; k < n; ++k) r = std::fma(a[k], b[k], r);
    return r;
}

inline int threads() {
#ifdef _OPENMP
    return g_threads > 0 ? g_threads : omp_get_max_threads();
#else
    return 1;
#endif
}

}  // namespace

extern "C" {

void orc_f16_to_f32(const uint16_t* in, float* out, int64_t n) {
    for (int64_t i = 0; i < n; ++i) out[i] = half_to_float(in[i]);
}
void orc_f32_to_f16(const float* in, uint16_t* out, int64_t n) {
    for (int64_t i = 0; i < n; ++i) out[i] = float_to_half(in[i]);
}
// software versions, exported so the tests can check the F16C path against them
void orc_f16_to_f32_sw(const uint16_t* in, float* out, int64_t n) {
    for (int64_t i = 0; i < n; ++i) out[i] = half_to_float_sw(in[i]);
}
void orc_f32_to_f16_sw(const float* in, uint16_t* out, int64_t n) {
    for (int64_t i = 0; i < n; ++i) out[i] = float_to_half_sw(in[i]);
}

void orc_set_dtype(int dtype) { g_dtype = dtype == 1 ? 1 : 0; }
int orc_get_dtype(void) { return g_dtype; }
void orc_bf16_to_f32(const uint16_t* in, float* out, int64_t n) {
    for (int64_t i = 0; i < n; ++i) out[i] = bf16_to_float(in[i]);
}
void orc_f32_to_bf16(const float* in, uint16_t* out, int64_t n) {
    for (int64_t i = 0; i < n; ++i) out[i] = float_to_bf16(in[i]);
}

int orc_num_threads(void) { return threads(); }
void orc_set_num_threads(int n) { g_threads = n; }

// A1 -- src/flash_attn/src/mask.h:139-229, softmax.h:66-91,239-256,
// flash_fwd_kernel.h:1266,1610-1615, flash_api.hpp:103.
// block_window_size > 0 adds the block-granular sliding window of the drafter's own layer
// (src/flash_attn/src/flash_blockmask.h:9,16,32,43-46 with kBlockN = 128,
// src/flash_attn/src/flash_fwd_launch_template.h:208; passed as Attention::window_size,
// src/model/attn.cuh:228): key blocks of 128 below
// ceil(P / 128) - block_window_size / 128 are not visited at all.
void orc_tree_attention_window(const uint16_t* q, const uint16_t* k, const uint16_t* v,
                               const uint64_t* mask, int T, int P, int Hq, int Hkv, int D,
                               int mask_words, int mask_k_range, int block_window_size, float scale,
                               uint16_t* out, float* lse) {
    const int S = P + T;
    const int kBlockN = 128;
    // flash_blockmask.h:9,16: q_block_idx = loop_step_idx (0) + seqlen_k - seqlen_q = P;  :32 k_window_left
    const int k_window_left = block_window_size > 0 ? (P + kBlockN - 1) / kBlockN - block_window_size / kBlockN : -1;
    const int first_key = k_window_left > 0 ? k_window_left * kBlockN : 0;
    const int Pm = S - mask_k_range;  // mask.h: mask_k_begin = seqlen_k - mask_k_range
    const int group = Hq / Hkv;
    // flash_api.hpp:103  scale_softmax_log2 = softmax_scale * M_LOG2E
    const float scale_log2 = scale * (float)M_LOG2E;
    std::vector<float> kf((size_t)S * D), vf((size_t)S * D);
    for (int g = 0; g < Hkv; ++g) {
        for (int c = 0; c < S; ++c) {
            const uint16_t* kr = k + ((size_t)c * Hkv + g) * D;
            const uint16_t* vr = v + ((size_t)c * Hkv + g) * D;
            for (int d = 0; d < D; ++d) {
                kf[(size_t)c * D + d] = h2f(kr[d]);
                vf[(size_t)c * D + d] = h2f(vr[d]);
            }
        }
        const int rows = group * T;
#pragma omp parallel num_threads(threads())
        {
            std::vector<float> s(S), qf(D), o(D);
#pragma omp for schedule(dynamic, 4)
            for (int r = 0; r < rows; ++r) {
                const int h = g * group + r / T;  // flash_fwd_kernel.h:1266 kv head = h / group
                const int i = r % T;
                const uint16_t* qr = q + ((size_t)i * Hq + h) * D;
                for (int d = 0; d < D; ++d) qf[d] = h2f(qr[d]);
                const uint64_t* mrow = mask + (size_t)i * mask_words;
                float m = -std::numeric_limits<float>::infinity();
                for (int c = 0; c < S; ++c) {
                    bool vis = true;
                    if (c >= Pm) {  // mask.h:187,194-198 mask bit of column c - mask_k_begin
                        int j = c - Pm;
                        vis = (mrow[j >> 6] >> (j & 63)) & 1ull;
                    }
                    if (c > P + i) vis = false;  // mask.h:185-186,199-203 causal: col < row + 1 + seqlen_k - seqlen_q
                    if (c < first_key) vis = false;  // flash_blockmask.h:43-46: blocks below k_window_left are skipped
                    if (vis) {
                        s[c] = dot_any(qf.data(), &kf[(size_t)c * D], D);
                        m = std::max(m, s[c]);
                    } else {
                        s[c] = -std::numeric_limits<float>::infinity();
                    }
                }
                // softmax.h:66-91: exp2f(x*scale_log2 - max*scale_log2); max=-inf -> 0
                const float max_scaled = (m == -std::numeric_limits<float>::infinity()) ? 0.f : m * scale_log2;
                float l = 0.f;
                for (int d = 0; d < D; ++d) o[d] = 0.f;
                for (int c = 0; c < S; ++c) {
                    if (s[c] == -std::numeric_limits<float>::infinity()) continue;
                    float p = exp2f(s[c] * scale_log2 - max_scaled);
                    l += p;  // row sum uses the fp32 p (softmax.h:157-200)
                    float ph = h2f(f2h(p));  // flash_fwd_kernel.h:1610 P -> fp16 before P.V
                    const float* vr = &vf[(size_t)c * D];
                    for (int d = 0; d < D; ++d) o[d] = std::fma(ph, vr[d], o[d]);
                }
                // softmax.h:239-256
                const bool bad = (l == 0.f || l != l);
                const float inv = bad ? 1.f : 1.f / l;
                uint16_t* orow = out + ((size_t)i * Hq + h) * D;
                for (int d = 0; d < D; ++d) orow[d] = f2h(o[d] * inv);
                if (lse) lse[(size_t)i * Hq + h] = bad ? std::numeric_limits<float>::infinity() : m * scale + logf(l);
            }
        }
    }
}

void orc_tree_attention(const uint16_t* q, const uint16_t* k, const uint16_t* v,
                        const uint64_t* mask, int T, int P, int Hq, int Hkv, int D,
                        int mask_words, int mask_k_range, float scale, uint16_t* out, float* lse) {
    orc_tree_attention_window(q, k, v, mask, T, P, Hq, Hkv, D, mask_words, mask_k_range, 0, scale, out, lse);
}

// a7 -- src/model/tree_drafter.cuh:79-86
void orc_gather_rows(const uint16_t* src, const int32_t* remap, int rows, int dim, uint16_t* dst) {
#pragma omp parallel for num_threads(threads()) schedule(static)
    for (int r = 0; r < rows; ++r)
        std::memcpy(dst + (size_t)r * dim, src + (size_t)remap[r] * dim, (size_t)dim * 2);
}

// a6 / a11 -- src/model/linear.cuh:8-37,82-101; elementwise.cuh:34-41
void orc_lm_head(const uint16_t* hid, const uint16_t* w, int n, int V, int H,
                 int apply_scale, float head_scale, uint16_t* logits) {
    std::vector<float> hf((size_t)n * H);
    const float sc = h2f(f2h(head_scale));  // scale is applied as a half (elementwise.cuh:34-41)
    for (size_t i = 0; i < (size_t)n * H; ++i) {
        float x = h2f(hid[i]);
        if (apply_scale) x = h2f(f2h(x * sc));  // linear.cuh:98 fp16 pre-scale
        hf[i] = x;
    }
#pragma omp parallel num_threads(threads())
    {
        std::vector<float> wf(H);
#pragma omp for schedule(static)
        for (int vv = 0; vv < V; ++vv) {
            const uint16_t* wr = w + (size_t)vv * H;
            for (int kk = 0; kk < H; ++kk) wf[kk] = h2f(wr[kk]);
            for (int r = 0; r < n; ++r)
                logits[(size_t)r * V + vv] = f2h(dot_any(&hf[(size_t)r * H], wf.data(), H));
        }
    }
}

// a8 -- src/model/eagle.cuh:29-89
void orc_log_softmax(uint16_t* x, int n, int dim, float* m_out, float* lse_out) {
    for (int r = 0; r < n; ++r) {
        uint16_t* row = x + (size_t)r * dim;
        float m = -std::numeric_limits<float>::infinity();
        for (int c = 0; c < dim; ++c) m = fmaxf(h2f(row[c]), m);
        float s = 0.f;
        for (int c = 0; c < dim; ++c) s += expf(h2f(row[c]) - m);
        const float ls = logf(s);
        for (int c = 0; c < dim; ++c) row[c] = f2h(h2f(row[c]) - m - ls);  // eagle.cuh:87
        if (m_out) m_out[r] = m;
        if (lse_out) lse_out[r] = ls;
    }
}

void orc_log_softmax_apply(uint16_t* x, int n, int dim, const float* m, const float* lse) {
    for (int r = 0; r < n; ++r) {
        uint16_t* row = x + (size_t)r * dim;
        for (int c = 0; c < dim; ++c) row[c] = f2h(h2f(row[c]) - m[r] - lse[r]);
    }
}

// a9 -- src/model/topk.cuh:17 ordering: v1 > v2 || (v1 == v2 && pos1 < pos2)
void orc_topk(const uint16_t* x, int n, int dim, int top, uint16_t* val, int32_t* pos) {
#pragma omp parallel for num_threads(threads()) schedule(static)
    for (int r = 0; r < n; ++r) {
        const uint16_t* row = x + (size_t)r * dim;
        std::vector<int32_t> idx(dim);
        std::iota(idx.begin(), idx.end(), 0);
        auto before = [row](int32_t a, int32_t b) {
            float va = h2f(row[a]), vb = h2f(row[b]);
            return va > vb || (va == vb && a < b);
        };
        std::partial_sort(idx.begin(), idx.begin() + top, idx.end(), before);
        for (int j = 0; j < top; ++j) {
            pos[(size_t)r * top + j] = idx[j];
            val[(size_t)r * top + j] = row[idx[j]];
        }
    }
}

// a10 -- src/model/tree_drafter.cuh:88-90
void orc_remap(const int32_t* in, int n, const int32_t* remap, int32_t* out) {
    for (int i = 0; i < n; ++i) out[i] = remap[in[i]];
}

// a12 -- cpmcu/speculative/tree_drafter.py:153,233; lowest index on ties
void orc_argmax(const uint16_t* logits, int n, int V, int32_t* gt) {
#pragma omp parallel for num_threads(threads()) schedule(static)
    for (int r = 0; r < n; ++r) {
        const uint16_t* row = logits + (size_t)r * V;
        float best = h2f(row[0]);
        int32_t bi = 0;
        for (int c = 1; c < V; ++c) {
            float x = h2f(row[c]);
            if (x > best) { best = x; bi = c; }
        }
        gt[r] = bi;
    }
}

// a13 -- src/model/tree_drafter.cuh:5-46
int orc_tree_accept(int T, int mask_words, const int32_t* pred, const int32_t* gt,
                    const int32_t* pos, int P, const uint64_t* mask, const int32_t* parent,
                    int32_t* best, int32_t* path) {
    uint64_t correct[4] = {1ull, 0, 0, 0};  // :9 bit 0 always set
    for (int i = 1; i < T; ++i)             // :10 pred[i] == gt[tree_parent[i]]
        if (pred[i] == gt[parent[i]]) correct[i >> 6] |= 1ull << (i & 63);
    int S = 64;
    while (S < T) S <<= 1;
    std::vector<int32_t> mx(S), mi(S);
    for (int i = 0; i < S; ++i) {           // :22-28
        bool full = i < T;
        if (full) {
            for (int w = 0; w < mask_words; ++w) {
                uint64_t mw = mask[(size_t)i * mask_words + w];
                if ((correct[w] & mw) != mw) { full = false; break; }
            }
        }
        if (full) { mx[i] = pos[i] - P + 1; mi[i] = i; }
        else      { mx[i] = 1;              mi[i] = 0; }
    }
    for (int off = S / 2; off > 0; off >>= 1)  // :30-36 strictly-greater tournament
        for (int i = 0; i < off; ++i)
            if (mx[i + off] > mx[i]) { mx[i] = mx[i + off]; mi[i] = mi[i + off]; }
    best[0] = mx[0];
    best[1] = mi[0];
    const int p = mi[0];
    for (int i = 0; i < T; ++i)                // :42-45
        if ((mask[(size_t)p * mask_words + (i >> 6)] >> (i & 63)) & 1ull) path[pos[i] - P] = i;
    return mx[0];
}

// a14 -- src/model/tree_drafter.cuh:48-77
void orc_kv_compact(uint16_t* const* caches, int num_caches, int row_halves, int P, int a,
                    const int32_t* path, const int32_t* gt, int32_t* ids_out) {
    std::vector<uint16_t> tmp((size_t)a * row_halves);
    for (int c = 0; c < num_caches; ++c) {
        uint16_t* cache = caches[c];
        for (int d = 0; d < a; ++d)  // kernel_1: stage
            std::memcpy(&tmp[(size_t)d * row_halves], cache + (size_t)(P + path[d]) * row_halves, (size_t)row_halves * 2);
        for (int d = 0; d < a; ++d)  // kernel_2: write back
            std::memcpy(cache + (size_t)(P + d) * row_halves, &tmp[(size_t)d * row_halves], (size_t)row_halves * 2);
    }
    if (ids_out)
        for (int d = 0; d < a; ++d) ids_out[d] = gt[path[d]];  // :74-76
}

// f2 -- rotary_embedding_kernel, src/model/rotary.cuh:7-34: in place on q [T][Hq][2*half] and k [T][Hkv][2*half].
// table (optional, [T][half][2]): use these (cos, sin) instead of computing them -- the staged form of
// the check, which takes the device's table and leaves only the rotation itself to compare.
void orc_rope(int T, int Hq, int Hkv, int half_dim, const float* inv_freq, const int32_t* pos, const float* table,
              uint16_t* q, uint16_t* k) {
    for (int t = 0; t < T; ++t) {
        const int p = pos ? pos[t] : 0;                                    // :10
        for (int pass = 0; pass < 2; ++pass) {
            uint16_t* x = pass == 0 ? q : k;
            const int heads = pass == 0 ? Hq : Hkv;
            for (int i = 0; i < heads * half_dim; ++i) {                   // :12 / :23
                const int row = i / half_dim, col = i % half_dim;
                const size_t offset = (size_t)t * heads * half_dim * 2 + (size_t)row * half_dim * 2;
                float cos_freq, sin_freq;
                if (table) {
                    cos_freq = table[((size_t)t * half_dim + col) * 2];
                    sin_freq = table[((size_t)t * half_dim + col) * 2 + 1];
                } else {
                    const float freq = (float)p * inv_freq[col];           // :16
                    cos_freq = cosf(freq);                                 // :17
                    sin_freq = sinf(freq);
                }
                const float a = h2f(x[offset + col]);
                const float b = h2f(x[offset + col + half_dim]);
                x[offset + col] = f2h(a * cos_freq - b * sin_freq);            // :20
                x[offset + col + half_dim] = f2h(a * sin_freq + b * cos_freq); // :21
            }
        }
    }
}

// f2/f3 -- the rest of MiniCPM4EagleImpl::verify after the acceptance, src/model/minicpm4/minicpm4_eagle.cuh:403-411,
// and the host side of the loop, cpmcu/speculative/tree_drafter.py:222,243-249.
//   prev_hidden[d] = hidden[path[d] / scale]      remap_hidden_kernel, src/model/eagle.cuh:108-115 (scale 1 at :404)
//   fix_kv_cache                                   orc_kv_compact
//   next_pos[d] = d + P                            make_arange_kernel, src/model/eagle.cuh:125-127, called with num_prev = a
//   result = (a, ids), *new_length = P + a, *next_root = ids[a - 1]
void orc_accept_commit(uint16_t* const* caches, int num_caches, int row_halves, int P, int a, const int32_t* path,
                       const int32_t* gt, const uint16_t* hidden, int hidden_dim, uint16_t* prev_hidden,
                       int32_t* next_pos, int32_t* result, int32_t* new_length, int32_t* next_root) {
    if (hidden)
        for (int d = 0; d < a; ++d) {
            const int real_row = path[d] / 1;
            for (int i = 0; i < hidden_dim; ++i) prev_hidden[(size_t)d * hidden_dim + i] = hidden[(size_t)real_row * hidden_dim + i];
        }
    orc_kv_compact(caches, num_caches, row_halves, P, a, path, gt, result + 1);
    result[0] = a;
    for (int d = 0; d < a; ++d) next_pos[d] = d + P;
    *new_length = P + a;
    *next_root = result[a];
}

// f1 -- d = 0 of draft(): src/model/minicpm4/minicpm4_eagle.cuh:319-332, init_tree src/model/eagle.cuh:91-93
void orc_draft_tree_begin(int k, const uint16_t* val, const int32_t* pos, const int32_t* token_id_remap,
                          uint16_t* tried_val, int32_t* tried_pos, uint16_t* cum, uint64_t* mask, int32_t* next_ids) {
    for (int i = 0; i < k; ++i) {
        tried_val[i] = val[i];                                     // :323
        tried_pos[i] = pos[i];                                     // :324
        next_ids[i] = token_id_remap ? token_id_remap[pos[i]] : pos[i];  // :325-329
        cum[i] = val[i];                                           // :330 topk_func_2->topk_val
        mask[i] = 1ull << i;                                       // eagle.cuh:92
    }
}

// f1 -- iteration d >= 1: src/model/minicpm4/minicpm4_eagle.cuh:367-382
void orc_draft_tree_extend(int k, int d, uint16_t* val, const int32_t* pos, const int32_t* token_id_remap,
                           uint16_t* tried_val, int32_t* tried_pos, int32_t* tried_parent, uint16_t* cum,
                           uint64_t* mask, int32_t* next_ids, int32_t* parent_rows) {
    const int kk = k * k;
    const int base = k + (d - 1) * kk;
    for (int i = 0; i < k; ++i)  // cumsum, eagle.cuh:103-106: half += half, rounded to half
        for (int j = 0; j < k; ++j) val[i * k + j] = f2h(h2f(val[i * k + j]) + h2f(cum[i]));
    for (int x = 0; x < kk; ++x) {  // :370-371
        tried_val[base + x] = val[x];
        tried_pos[base + x] = pos[x];
    }
    std::vector<uint16_t> v2(k);
    std::vector<int32_t> p2(k);
    orc_topk(val, 1, kk, k, v2.data(), p2.data());  // :372
    std::vector<uint64_t> tmp(mask, mask + k);      // :374
    for (int i = 0; i < k; ++i) {
        tried_parent[(d - 1) * k + i] = p2[i] + base;               // :375, eagle.cuh:95-97
        mask[i] = tmp[p2[i] / k] | (1ull << (k * d + i));           // :376, eagle.cuh:99-101
        parent_rows[i] = p2[i] / k;                                 // :377 remap_hidden's row
        const int32_t fr = pos[p2[i]];                              // :378-382, eagle.cuh:121-127
        next_ids[i] = token_id_remap ? token_id_remap[fr] : fr;
        cum[i] = v2[i];
    }
}

// f1 -- final selection and tree: src/model/minicpm4/minicpm4_eagle.cuh:385-393, eagle.cuh:188-214
void orc_draft_tree_finish(int k, int num_iter, int T, int P, const int32_t* token_id_remap,
                           const uint16_t* tried_val, const int32_t* tried_pos, const int32_t* tried_parent,
                           int32_t* ids_out, int32_t* tree_pos, uint64_t* tree_mask, int32_t* tree_parent) {
    const int kk = k * k;
    const int total = k + (num_iter - 1) * kk;
    const int W = (T + 63) / 64;
    std::vector<uint16_t> v3(T - 1);
    std::vector<int32_t> sel(T - 1);
    orc_topk(tried_val, 1, total, T - 1, v3.data(), sel.data());  // :385
    std::vector<int32_t> reverse(total, 0);
    for (int i = 1; i < T; ++i) reverse[sel[i - 1]] = i;          // eagle.cuh:191-193
    for (int w = 0; w < W; ++w) tree_mask[w] = 0;
    tree_mask[0] = 1;                                             // :196
    tree_pos[0] = P;                                              // :197
    tree_parent[0] = 0;
    for (int i = 1; i < T; ++i) {
        int p = sel[i - 1];
        tree_pos[i] = P + (p < k ? 1 : (p - k) / kk + 2);         // :200
        if (p < k) {
            p = -1;
        } else {
            p -= k;
            p = p < kk ? p / k : tried_parent[(p - kk) / k];      // :203-211
        }
        const int parent = p == -1 ? 0 : reverse[p];              // :212
        tree_parent[i] = parent;
        for (int w = 0; w < W; ++w) tree_mask[(size_t)i * W + w] = tree_mask[(size_t)parent * W + w];  // :214
        tree_mask[(size_t)i * W + (i >> 6)] |= 1ull << (i & 63);  // :201
        const int32_t fr = tried_pos[sel[i - 1]];                 // :389-393
        ids_out[i] = token_id_remap ? token_id_remap[fr] : fr;
    }
}

}  // extern "C"
