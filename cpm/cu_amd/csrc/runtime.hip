// Host runtime of libcpmcu_amd: error plumbing, the library stream, and the model-level mirror of
// the reference's pybind module (src/entry.cu:98-534) for the verify/draft path: one process-global
// model that owns the lm_head, the FR-Spec sub-matrix, the paged KV pools of every layer, one page
// table and scratch.
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <initializer_list>
#include <map>
#include <utility>
#include <string>
#include <vector>

#include "common.h"
#include "internal.h"

namespace cpmcu {

namespace {
thread_local std::string g_error;
hipStream_t g_stream = nullptr;
}  // namespace

void set_error(const char* fmt, ...) {
    char buf[1024];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    g_error = buf;
}

hipStream_t resolve_stream(void* stream) {
    if (stream) return (hipStream_t)stream;
    if (!g_stream) {
        // a blocking stream, like the reference's calc_stream (src/utils.cu:19): work on the legacy
        // default stream is implicitly ordered with it
        if (hipStreamCreate(&g_stream) != hipSuccess) g_stream = nullptr;
    }
    return g_stream;
}

Options& options() {
    static Options opt = [] {
        Options o;
        if (const char* e = getenv("CPMCU_ATTN_KV_GROUPS")) {
            if (e[0] == '1' && e[1] == 0) o.attn_kv_groups = 1;
            if (e[0] == '2' && e[1] == 0) o.attn_kv_groups = 2;
        }
        if (getenv("CPMCU_HEAD_NO_SHARE") != nullptr) o.head_share_last_pass = 0;
        if (getenv("CPMCU_HEAD_NO_STREAM") != nullptr) o.head_stream_kernel = 0;
        if (getenv("CPMCU_ATTN_SEPARATE_MERGE") != nullptr) o.attn_merge_in_launch = 0;
        return o;
    }();
    return opt;
}

namespace {

struct PerfEntry {
    double ms = 0;
    long count = 0;
};

struct Model {
    // base model geometry (init_base_model)
    bool base = false;
    float memory_limit = 0.f;
    int vocab = 0, layers = 0, hidden = 0, q_heads = 0, kv_heads = 0, head_dim = 0;
    float scale_lmhead = 1.f;
    int dtype = 0;  // 0 = fp16, 1 = bf16
    // drafter (init_eagle_model / init_minicpm4_eagle_model)
    bool drafter = false;
    int num_iter = 0, topk_per_iter = 0, tree_size = 0, frspec_vocab = 0;
    int draft_layers = 0;   // the drafter's own transformer layers: their KV pools follow the base model's
    int eagle_window = 0;   // block sliding window of those layers, in tokens (0 = none)
    // storage
    bool storage = false;
    int num_pages = 0;
    f16* lm_head = nullptr;
    f16* fr_head = nullptr;  // == lm_head when FR-Spec is off
    int32_t* token_id_remap = nullptr;
    bool remap_loaded = false, lm_head_loaded = false;
    std::vector<void*> k_pools, v_pools;
    void** d_k_pools = nullptr;
    void** d_v_pools = nullptr;
    int32_t* block_table = nullptr;
    void* attn_ws = nullptr;
    size_t attn_ws_bytes = 0;
    void* head_ws = nullptr;
    size_t head_ws_bytes = 0;
    f16* draft_logits = nullptr;  // [16][frspec_vocab]
    float* row_stats = nullptr;   // [16][2]
    // the drafter's tree bookkeeping between the rounds of one draft (tried_history_*, eagle_mask_2d and the
    // running log-probs of src/model/minicpm4/minicpm4_eagle.cuh:158-170) and the head's top-k of the round
    void* draft_state = nullptr;
    f16* topk_val = nullptr;      // [16][topk_per_iter]
    int32_t* topk_pos = nullptr;  // [16][topk_per_iter]
    int32_t* topk_ids = nullptr;  // [16][topk_per_iter]
    int draft_rounds_done = 0;    // rounds of the current draft that have run (0 .. num_iter)
    int32_t* d_best = nullptr;
    int32_t* d_ids = nullptr;     // [64] accepted ids of the last verify
    int32_t* h_result = nullptr;  // pinned, device-visible: (a, ids) of the last verify
    uint64_t* chain_mask = nullptr;
    bool perf = false;
    std::map<std::string, PerfEntry> perf_log;
    // captured verify steps, keyed like the reference's decode graph (src/entry.cu:475-492) on
    // (padded_length, num_tokens); the signature covers every address baked into the graph
    struct StepGraph {
        hipGraph_t graph = nullptr;
        hipGraphExec_t exec = nullptr;
        uint64_t signature = 0;
        unsigned long long last_use = 0;
    };
    unsigned long long graph_clock = 0;
    std::map<std::pair<int, int>, std::vector<StepGraph>> step_graphs;
    // sequences of model-level calls captured by the caller (cpmcu_capture_begin / _end)
    std::vector<StepGraph> user_graphs;
    bool capturing = false;
};

Model* g_model = nullptr;
constexpr int kMaxStepGraphs = 16;  // captured verify steps kept at a time (least recently used goes first)

int require_model(bool need_storage) {
    if (!g_model || !g_model->base) {
        set_error("no model: call init_base_model first");
        return CPMCU_ERR_RUNTIME;
    }
    if (need_storage && !g_model->storage) {
        set_error("storage not initialised: call init_storage first");
        return CPMCU_ERR_RUNTIME;
    }
    return CPMCU_OK;
}

struct PerfScope {
    const char* label;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    hipStream_t st;
    PerfScope(const char* l, hipStream_t s) : label(l), st(s) {
        if (g_model && g_model->perf && !g_model->capturing) {  // (a capture records launches, it does not run them)
            (void)hipEventCreate(&e0);
            (void)hipEventCreate(&e1);
            (void)hipEventRecord(e0, st);
        }
    }
    ~PerfScope() {
        if (e0) {
            (void)hipEventRecord(e1, st);
            (void)hipEventSynchronize(e1);  // the reference's timers synchronise on stop too (src/perf.cuh:139-166)
            float ms = 0;
            (void)hipEventElapsedTime(&ms, e0, e1);
            auto& ent = g_model->perf_log[label];
            ent.ms += ms;
            ent.count += 1;
            (void)hipEventDestroy(e0);
            (void)hipEventDestroy(e1);
        }
    }
};

// Synchronises the stream and looks at what attention launches left behind for the host (the report words travel to
// pinned memory in front of the synchronisation: no round trip of their own): a length outside what the host had
// promised is an error; merge waits that ran out are counted for the summary.
long g_abandoned_waits = 0;
// Fused FR-Spec launches: rows finished from the published candidates, rows redone from the logits, waits that ran out.
long g_frspec_fused_rows = 0, g_frspec_slow_rows = 0, g_frspec_timeouts = 0;
int synchronize_and_check(hipStream_t st) {
    int rc = attention_report_enqueue(st);
    if (rc) return rc;
    rc = head_fuse_report_enqueue(st);
    if (rc) return rc;
    CPMCU_HIP(hipStreamSynchronize(st));
    int bad = 0;
    unsigned int abandoned = 0;
    rc = attention_report_take(&bad, &abandoned);
    if (rc) return rc;
    g_abandoned_waits += abandoned;
    unsigned int fr_timeouts = 0, fr_slow = 0, fr_fused = 0;
    rc = head_fuse_report_take(&fr_timeouts, &fr_slow, &fr_fused);
    if (rc) return rc;
    g_frspec_fused_rows += fr_fused;
    g_frspec_slow_rows += fr_slow;
    g_frspec_timeouts += fr_timeouts;
    if (fr_timeouts != 0) {
        set_error("%u row(s) of a one-launch FR-Spec head were not finished: the workgroups of the launch were not all resident within "
                  "the wait (frspec_wait_us); those rows hold index -1, and the head runs as two launches from now on", fr_timeouts);
        return CPMCU_ERR_RUNTIME;
    }
    if (bad != 0) {
        set_error("a tree-attention launch read a KV length of %d from device memory, outside [rows, max_kv_len] of its call; "
                  "it ran on the clamped length and its output is not valid", bad < 0 ? 0 : bad);
        return CPMCU_ERR_RUNTIME;
    }
    return CPMCU_OK;
}

int check_dtype(int torch_dtype) {
    if (torch_dtype != 0 && torch_dtype != 1) {  // 0 = fp16, 1 = bf16 (cpmcu/llm.py:11-14)
        set_error("dtype %d is not compiled into this library (0 = fp16, 1 = bf16)", torch_dtype);
        return CPMCU_ERR_RUNTIME;  // std::runtime_error in the reference, src/entry.cu:43,52
    }
    return CPMCU_OK;
}

}  // namespace
}  // namespace cpmcu

using namespace cpmcu;

extern "C" const char* cpmcu_last_error(void) { return g_error.c_str(); }
extern "C" const char* cpmcu_version(void) { return "cpmcu_amd 0.1 (gfx950)"; }

extern "C" int cpmcu_set_option(const char* name, int value) {
    CPMCU_CHECK_ARG(name, "set_option: null name");
    const std::string nm(name);
    if (nm == "dtype") {
        // the element type of the 16-bit tensors the operator-level entry points are handed from now on (the model-level
        // ones follow cpmcu_init_base_model's torch_dtype, which sets the same switch)
        CPMCU_CHECK_ARG(value == 0 || value == 1, "set_option: dtype=%d must be 0 (fp16) or 1 (bf16)", value);
        options().dtype = value;
    } else if (nm == "attn_kv_groups") {
        CPMCU_CHECK_ARG(value >= 0 && value <= 2, "set_option: attn_kv_groups=%d outside [0, 2]", value);
        options().attn_kv_groups = value;
    } else if (nm == "head_stream_kernel") {
        CPMCU_CHECK_ARG(value == 0 || value == 1, "set_option: head_stream_kernel=%d must be 0 or 1", value);
        options().head_stream_kernel = value;
    } else if (nm == "head_share_last_pass") {
        CPMCU_CHECK_ARG(value == 0 || value == 1, "set_option: head_share_last_pass=%d must be 0 or 1", value);
        options().head_share_last_pass = value;
    } else if (nm == "attn_merge_wait_us") {
        CPMCU_CHECK_ARG(value >= 0 && value <= 1000000, "set_option: attn_merge_wait_us=%d outside [0, 1000000]", value);
        options().attn_merge_wait_us = value;
    } else if (nm == "attn_merge_in_launch") {
        CPMCU_CHECK_ARG(value == 0 || value == 1, "set_option: attn_merge_in_launch=%d must be 0 or 1", value);
        options().attn_merge_in_launch = value;
        if (value) attention_merge_reenable();  // also for workspaces that went back to the combine launch after an abandoned wait
    } else if (nm == "frspec_fused") {
        CPMCU_CHECK_ARG(value == 0 || value == 1, "set_option: frspec_fused=%d must be 0 or 1", value);
        options().frspec_fused = value;
        if (value) head_fuse_reenable();  // also after a wait that ran out
    } else if (nm == "topk_row_kernel") {
        CPMCU_CHECK_ARG(value == 0 || value == 1, "set_option: topk_row_kernel=%d must be 0 or 1", value);
        options().topk_row_kernel = value;
    } else if (nm == "frspec_wait_us") {
        CPMCU_CHECK_ARG(value >= 0 && value <= 1000000, "set_option: frspec_wait_us=%d outside [0, 1000000]", value);
        options().frspec_wait_us = value;
    } else {
        set_error("set_option: unknown option %s", name);
        return CPMCU_ERR_INVALID_ARGUMENT;
    }
    return CPMCU_OK;
}

extern "C" int cpmcu_init_base_model(float memory_limit, int vocab_size, int num_hidden_layers, int hidden_size,
                                     int intermediate_size, int num_attention_heads, int num_key_value_heads,
                                     int head_dim, float rms_norm_eps, int torch_dtype, int chunk_length,
                                     float scale_embed, float scale_lmhead, float scale_residual) {
    (void)intermediate_size; (void)rms_norm_eps; (void)chunk_length; (void)scale_embed; (void)scale_residual;
    int rc = check_dtype(torch_dtype);
    if (rc) return rc;
    CPMCU_CHECK_ARG(memory_limit > 0.f && memory_limit <= 1.f, "init_base_model: memory_limit=%g outside (0, 1]", memory_limit);
    CPMCU_CHECK_ARG(vocab_size > 0 && num_hidden_layers > 0 && hidden_size > 0, "init_base_model: bad model shape");
    CPMCU_CHECK_ARG(head_dim == kHeadDim, "init_base_model: head_dim=%d, this library is built for %d", head_dim, kHeadDim);
    CPMCU_CHECK_ARG(num_key_value_heads > 0 && num_attention_heads % num_key_value_heads == 0,
                    "init_base_model: %d attention heads not a multiple of %d kv heads", num_attention_heads, num_key_value_heads);
    if (g_model) cpmcu_shutdown();
    g_model = new Model();
    Model& m = *g_model;
    m.base = true;
    m.memory_limit = memory_limit;
    m.vocab = vocab_size;
    m.layers = num_hidden_layers;
    m.hidden = hidden_size;
    m.q_heads = num_attention_heads;
    m.kv_heads = num_key_value_heads;
    m.head_dim = head_dim;
    m.scale_lmhead = scale_lmhead;
    m.dtype = torch_dtype;
    options().dtype = torch_dtype;  // the model's element type is the process's: every kernel launch reads this switch
    const char* pe = getenv("CPMCU_PERF");
    m.perf = pe && pe[0] == '1';
    return CPMCU_OK;
}

extern "C" int cpmcu_init_eagle_model(int num_layers, int num_iter, int topk_per_iter, int tree_size, int torch_dtype) {
    return cpmcu_init_minicpm4_eagle_model(num_layers, num_iter, topk_per_iter, tree_size, torch_dtype, 0, 0, 0, 0, 1.f, 1, 1);
}

extern "C" int cpmcu_init_minicpm4_eagle_model(int num_layers, int num_iter, int topk_per_iter, int tree_size,
                                               int torch_dtype, int apply_eagle_quant, int group_size,
                                               int eagle_window_size, int frspec_vocab_size, float residual_scale,
                                               int use_input_norm, int use_attn_norm) {
    (void)group_size; (void)residual_scale; (void)use_input_norm; (void)use_attn_norm;
    int rc = require_model(false);
    if (rc) return rc;
    rc = check_dtype(torch_dtype);
    if (rc) return rc;
    CPMCU_CHECK_ARG(torch_dtype == g_model->dtype, "init_minicpm4_eagle_model: dtype %d differs from the base model's %d", torch_dtype,
                    g_model->dtype);
    if (apply_eagle_quant) {
        set_error("init_minicpm4_eagle_model: quantised EAGLE layers are outside the verify/draft path");
        return CPMCU_ERR_UNSUPPORTED;
    }
    Model& m = *g_model;
    CPMCU_CHECK_ARG(!m.storage, "init_minicpm4_eagle_model: storage already initialised");
    // the reference asserts tree_size <= 64 at this boundary (src/model/minicpm4/minicpm4_eagle.cuh:69)
    CPMCU_CHECK_ARG(tree_size >= 1 && tree_size <= 64, "init_minicpm4_eagle_model: tree_size=%d outside [1, 64]", tree_size);
    CPMCU_CHECK_ARG(num_iter >= 1 && topk_per_iter >= 1 && topk_per_iter <= tree_size - 1 && topk_per_iter <= 16,
                    "init_minicpm4_eagle_model: topk_per_iter=%d must be in [1, min(16, tree_size-1)]", topk_per_iter);
    CPMCU_CHECK_ARG(frspec_vocab_size >= 0 && frspec_vocab_size <= m.vocab, "init_minicpm4_eagle_model: frspec_vocab_size=%d", frspec_vocab_size);
    CPMCU_CHECK_ARG(num_layers >= 0 && num_layers <= 64, "init_minicpm4_eagle_model: num_layers=%d outside [0, 64]", num_layers);
    CPMCU_CHECK_ARG(eagle_window_size == 0 || eagle_window_size >= 128,
                    "init_minicpm4_eagle_model: eagle_window_size=%d must be 0 or at least one block of 128", eagle_window_size);
    m.drafter = true;
    m.draft_layers = num_layers;
    m.eagle_window = eagle_window_size;
    m.num_iter = num_iter;
    m.topk_per_iter = topk_per_iter;
    m.tree_size = tree_size;
    m.frspec_vocab = frspec_vocab_size > 0 ? frspec_vocab_size : m.vocab;
    return CPMCU_OK;
}

namespace {

void destroy_step_graphs(Model& m) {
    for (auto& kv : m.step_graphs)
        for (auto& g : kv.second) {
            if (g.exec) (void)hipGraphExecDestroy(g.exec);
            if (g.graph) (void)hipGraphDestroy(g.graph);
        }
    m.step_graphs.clear();
    for (auto& g : m.user_graphs) {
        if (g.exec) (void)hipGraphExecDestroy(g.exec);
        if (g.graph) (void)hipGraphDestroy(g.graph);
    }
    m.user_graphs.clear();
}

// Frees everything init_storage allocates and forgets it (also after a failure half-way, so that a retry starts clean).
void release_storage(Model& m) {
    destroy_step_graphs(m);
    if (m.fr_head && m.fr_head != m.lm_head) (void)hipFree(m.fr_head);
    (void)hipFree(m.lm_head);
    (void)hipFree(m.token_id_remap);
    for (void* p : m.k_pools) (void)hipFree(p);
    for (void* p : m.v_pools) (void)hipFree(p);
    (void)hipFree(m.d_k_pools);
    (void)hipFree(m.d_v_pools);
    (void)hipFree(m.block_table);
    if (m.attn_ws) attention_release_workspace(m.attn_ws);
    if (m.head_ws) head_fuse_release_workspace(m.head_ws);
    (void)hipFree(m.attn_ws);
    (void)hipFree(m.head_ws);
    (void)hipFree(m.draft_logits);
    (void)hipFree(m.row_stats);
    (void)hipFree(m.draft_state);
    (void)hipFree(m.topk_val);
    (void)hipFree(m.topk_pos);
    (void)hipFree(m.topk_ids);
    (void)hipFree(m.d_best);
    (void)hipFree(m.d_ids);
    (void)hipFree(m.chain_mask);
    if (m.h_result) (void)hipHostFree(m.h_result);
    m.lm_head = m.fr_head = nullptr;
    m.token_id_remap = nullptr;
    m.k_pools.clear();
    m.v_pools.clear();
    m.d_k_pools = m.d_v_pools = nullptr;
    m.block_table = nullptr;
    m.attn_ws = m.head_ws = m.draft_state = nullptr;
    m.draft_logits = nullptr;
    m.row_stats = nullptr;
    m.topk_val = nullptr;
    m.topk_pos = m.topk_ids = nullptr;
    m.d_best = m.d_ids = m.h_result = nullptr;
    m.chain_mask = nullptr;
    m.storage = m.remap_loaded = m.lm_head_loaded = false;
    m.num_pages = 0;
}

int init_storage_impl(Model& m, int* max_context);

}  // namespace

extern "C" int cpmcu_init_storage(int* max_context) {
    int rc = require_model(false);
    if (rc) return rc;
    Model& m = *g_model;
    CPMCU_CHECK_ARG(!m.storage, "init_storage: already initialised");
    rc = init_storage_impl(m, max_context);
    if (rc) release_storage(m);  // nothing of a failed attempt stays allocated
    return rc;
}

namespace {

int init_storage_impl(Model& m, int* max_context) {
    int rc = CPMCU_OK;
    size_t free_b = 0, total_b = 0;
    CPMCU_HIP(hipMemGetInfo(&free_b, &total_b));
    const size_t budget = (size_t)((double)total_b * m.memory_limit);
    size_t used = 0;
    auto alloc = [&](void** ptr, size_t bytes) -> int {
        bytes = align_up(bytes, 256);
        if (used + bytes > budget || bytes > free_b) {
            set_error("init_storage: out of memory budget (%zu + %zu > %zu bytes)", used, bytes, budget);
            return CPMCU_ERR_RUNTIME;
        }
        CPMCU_HIP(hipMalloc(ptr, bytes));
        used += bytes;
        return CPMCU_OK;
    };
    const int max_tree = kMaxTree;  // decode_attention / draft_attention accept up to 64 rows whatever the tree size, verify_step up to kMaxTree
    if ((rc = alloc((void**)&m.lm_head, cpmcu_head_weight_tiled_bytes(m.vocab, m.hidden)))) return rc;  // kept in tiled layout
    if (m.drafter && m.frspec_vocab != m.vocab) {
        if ((rc = alloc((void**)&m.fr_head, cpmcu_head_weight_tiled_bytes(m.frspec_vocab, m.hidden)))) return rc;
        if ((rc = alloc((void**)&m.token_id_remap, (size_t)m.frspec_vocab * 4))) return rc;
    } else {
        m.fr_head = m.lm_head;
    }
    m.head_ws_bytes = cpmcu_head_workspace_bytes(128, m.vocab);
    if ((rc = alloc(&m.head_ws, m.head_ws_bytes))) return rc;
    if (m.drafter) {
        if ((rc = alloc((void**)&m.draft_logits, (size_t)16 * m.frspec_vocab * 2))) return rc;
        if ((rc = alloc((void**)&m.row_stats, 16 * 2 * sizeof(float)))) return rc;
        if ((rc = alloc(&m.draft_state, cpmcu_draft_tree_state_bytes(m.topk_per_iter, m.num_iter)))) return rc;
        if ((rc = alloc((void**)&m.topk_val, (size_t)16 * m.topk_per_iter * sizeof(f16)))) return rc;
        if ((rc = alloc((void**)&m.topk_pos, (size_t)16 * m.topk_per_iter * sizeof(int32_t)))) return rc;
        if ((rc = alloc((void**)&m.topk_ids, (size_t)16 * m.topk_per_iter * sizeof(int32_t)))) return rc;
        // the state of the one-launch draft head is assigned now, ahead of any captured launch
        (void)cpmcu_frspec_head_mode(m.head_ws, CPMCU_W_TILED, 1, m.frspec_vocab, m.hidden, m.topk_per_iter);
    }
    if ((rc = alloc((void**)&m.d_best, 2 * sizeof(int32_t)))) return rc;
    if ((rc = alloc((void**)&m.d_ids, 64 * sizeof(int32_t)))) return rc;
    CPMCU_HIP(hipHostMalloc((void**)&m.h_result, (1 + 64) * sizeof(int32_t), hipHostMallocDefault));
    if ((rc = alloc((void**)&m.chain_mask, 64 * sizeof(uint64_t)))) return rc;
    {
        uint64_t rows[64];
        for (int i = 0; i < 64; ++i) rows[i] = i == 63 ? ~0ull : ((2ull << i) - 1ull);
        CPMCU_HIP(hipMemcpy(m.chain_mask, rows, sizeof(rows), hipMemcpyHostToDevice));
    }
    // load_model passes lm_head.weight through a row-major staging buffer of its full size: keep room for it
    used += align_up((size_t)m.vocab * m.hidden * sizeof(f16), 256);
    // KV pools take what is left of the budget, in whole pages (the reference gives the KV cache
    // all remaining pool memory, src/model/kvcache.cuh:50).
    const size_t page_bytes = (size_t)m.kv_heads * kPage * kHeadDim * 2;  // one of K/V, one layer
    const int all_layers = m.layers + m.draft_layers;  // the drafter's layers keep caches of the same length (src/model/minicpm4/minicpm4_eagle.cuh:76,183-184)
    const size_t per_page_all = page_bytes * 2 * all_layers + sizeof(int32_t);  // + the page's block-table entry
    const size_t remaining = budget > used ? budget - used : 0;
    const size_t free_now = free_b > used ? free_b - used : 0;
    size_t pages = std::min(remaining, (size_t)(free_now * 0.95)) / per_page_all;
    if (pages > (1u << 20)) pages = 1u << 20;
    if (pages < 1) {
        set_error("init_storage: memory budget leaves no room for a KV page");
        return CPMCU_ERR_RUNTIME;
    }
    // attention scratch is sized once the context bound is known; take it out of the page count
    m.attn_ws_bytes = cpmcu_tree_attention_workspace_bytes(max_tree, m.q_heads, m.kv_heads, (int)std::min<size_t>(pages * kPage, 1u << 30));
    const size_t ws_pages = ceil_div((int)(m.attn_ws_bytes / 1024), (int)(per_page_all / 1024)) + 1;
    if (pages <= ws_pages) {
        set_error("init_storage: memory budget too small for the attention workspace");
        return CPMCU_ERR_RUNTIME;
    }
    pages -= ws_pages;
    CPMCU_HIP(hipMalloc(&m.attn_ws, m.attn_ws_bytes));
    // the state of the in-launch merge is made now, ahead of any captured launch
    attention_prepare_workspace(m.attn_ws, nullptr);
    m.num_pages = (int)pages;
    m.k_pools.assign(all_layers, nullptr);
    m.v_pools.assign(all_layers, nullptr);
    for (int l = 0; l < all_layers; ++l) {
        CPMCU_HIP(hipMalloc(&m.k_pools[l], page_bytes * pages));
        CPMCU_HIP(hipMalloc(&m.v_pools[l], page_bytes * pages));
        CPMCU_HIP(hipMemset(m.k_pools[l], 0, page_bytes * pages));
        CPMCU_HIP(hipMemset(m.v_pools[l], 0, page_bytes * pages));
    }
    CPMCU_HIP(hipMalloc((void**)&m.d_k_pools, m.layers * sizeof(void*)));
    CPMCU_HIP(hipMalloc((void**)&m.d_v_pools, m.layers * sizeof(void*)));
    CPMCU_HIP(hipMemcpy(m.d_k_pools, m.k_pools.data(), m.layers * sizeof(void*), hipMemcpyHostToDevice));
    CPMCU_HIP(hipMemcpy(m.d_v_pools, m.v_pools.data(), m.layers * sizeof(void*), hipMemcpyHostToDevice));
    CPMCU_HIP(hipMalloc((void**)&m.block_table, pages * sizeof(int32_t)));
    {
        std::vector<int32_t> ident(pages);
        for (size_t i = 0; i < pages; ++i) ident[i] = (int32_t)i;
        CPMCU_HIP(hipMemcpy(m.block_table, ident.data(), pages * sizeof(int32_t), hipMemcpyHostToDevice));
    }
    m.storage = true;
    if (max_context) *max_context = (int)std::min<size_t>(pages * kPage, 0x7fffffff);
    return CPMCU_OK;
}

}  // namespace

// Extension (no reference counterpart): install a logical -> physical page permutation.
extern "C" int cpmcu_set_block_table(const int32_t* host_table, int n) {
    int rc = require_model(true);
    if (rc) return rc;
    Model& m = *g_model;
    CPMCU_CHECK_ARG(!m.capturing, "set_block_table copies synchronously: it cannot be part of a capture");
    CPMCU_CHECK_ARG(host_table && n >= 1 && n <= m.num_pages, "set_block_table: n=%d outside [1, %d]", n, m.num_pages);
    std::vector<char> seen(m.num_pages, 0);
    for (int i = 0; i < n; ++i) {
        CPMCU_CHECK_ARG(host_table[i] >= 0 && host_table[i] < m.num_pages && !seen[host_table[i]],
                        "set_block_table: entry %d = %d is out of range or repeated", i, host_table[i]);
        seen[host_table[i]] = 1;
    }
    // The logical pages behind the n given ones take the physical pages that are left, in ascending order: the table
    // stays a permutation of all pages, so a context that grows past the given prefix never lands on a page twice.
    std::vector<int32_t> full(host_table, host_table + n);
    for (int pg = 0; pg < m.num_pages; ++pg)
        if (!seen[pg]) full.push_back(pg);
    CPMCU_HIP(hipStreamSynchronize(resolve_stream(nullptr)));
    CPMCU_HIP(hipMemcpy(m.block_table, full.data(), full.size() * sizeof(int32_t), hipMemcpyHostToDevice));
    return CPMCU_OK;
}

extern "C" int cpmcu_load_model(const char* name, uint64_t host_ptr) {
    int rc = require_model(true);
    if (rc) return rc;
    Model& m = *g_model;
    CPMCU_CHECK_ARG(name && host_ptr, "load_model: null argument");
    const std::string nm(name);
    hipStream_t st = resolve_stream(nullptr);
    if (nm.rfind("eagle.token_id_remap", 0) == 0) {  // src/model/minicpm4/minicpm4_eagle.cuh:193-194
        CPMCU_CHECK_ARG(m.drafter && m.token_id_remap, "load_model: %s given but FR-Spec is not configured", name);
        CPMCU_HIP(hipMemcpy(m.token_id_remap, (const void*)host_ptr, (size_t)m.frspec_vocab * 4, hipMemcpyHostToDevice));
        m.remap_loaded = true;
        return CPMCU_OK;
    }
    if (nm.rfind("lm_head", 0) == 0) {  // src/model/model.cuh:116-137 routing by prefix
        if (m.fr_head != m.lm_head && !m.remap_loaded) {
            set_error("load_model: eagle.token_id_remap must be loaded before lm_head.weight");
            return CPMCU_ERR_RUNTIME;
        }
        // The row-major matrix only passes through a staging buffer: both heads are kept in the tiled
        // layout their kernels stream fastest; the FR-Spec gather (remap_copy,
        // src/model/minicpm4/minicpm4_eagle.cuh:215-219) is fused into its re-tiling.
        void* staging = nullptr;
        CPMCU_HIP(hipMalloc(&staging, (size_t)m.vocab * m.hidden * 2));
        rc = CPMCU_OK;
        if (hipMemcpy(staging, (const void*)host_ptr, (size_t)m.vocab * m.hidden * 2, hipMemcpyHostToDevice) != hipSuccess) {
            set_error("load_model: copy of lm_head.weight to the device failed");
            rc = CPMCU_ERR_HIP;
        }
        if (!rc) rc = cpmcu_head_weight_tile(staging, nullptr, m.vocab, m.hidden, m.lm_head, st);
        if (!rc && m.fr_head != m.lm_head) rc = cpmcu_head_weight_tile(staging, m.token_id_remap, m.frspec_vocab, m.hidden, m.fr_head, st);
        if (!rc && hipStreamSynchronize(st) != hipSuccess) {
            set_error("load_model: re-tiling of lm_head.weight failed");
            rc = CPMCU_ERR_HIP;
        }
        (void)hipFree(staging);
        if (rc) return rc;
        m.lm_head_loaded = true;
        return CPMCU_OK;
    }
    set_error("Unsupported name: %s (only lm_head.weight and eagle.token_id_remap belong to the verify/draft path)", name);
    return CPMCU_ERR_INVALID_ARGUMENT;  // std::invalid_argument, src/model/model.cuh:131-135
}

extern "C" int cpmcu_prefill(int, int, uint64_t, uint64_t, uint64_t) {
    set_error("prefill runs the dense transformer layers, which are outside the verify/draft path of this library");
    return CPMCU_ERR_UNSUPPORTED;
}

extern "C" int cpmcu_decode(int, int, uint64_t, uint64_t, uint64_t, uint64_t, uint64_t, int) {
    set_error("decode runs the dense transformer layers, which are outside the verify/draft path of this library; "
              "use decode_attention and decode_lm_head for the parts that are on it");
    return CPMCU_ERR_UNSUPPORTED;
}

extern "C" int cpmcu_draft(uint64_t, uint64_t, uint64_t, uint64_t, uint64_t) {
    set_error("draft runs the EAGLE decoder layer, which is outside the verify/draft path of this library; "
              "use draft_head for the FR-Spec head + top-k that is on it");
    return CPMCU_ERR_UNSUPPORTED;
}

extern "C" int cpmcu_decode_attention(int layer, int input_length, int padded_length, uint64_t q, uint64_t k_new,
                                      uint64_t v_new, uint64_t cache_length, uint64_t mask_2d, uint64_t out) {
    int rc = require_model(true);
    if (rc) return rc;
    Model& m = *g_model;
    CPMCU_CHECK_ARG(layer >= 0 && layer < m.layers, "decode_attention: layer %d outside [0, %d)", layer, m.layers);
    CPMCU_CHECK_ARG(input_length >= 1 && input_length <= 64, "decode_attention: input_length=%d outside [1, 64]", input_length);
    CPMCU_CHECK_ARG(padded_length >= input_length && padded_length <= m.num_pages * kPage,
                    "decode_attention: padded_length=%d outside [%d, %d]", padded_length, input_length, m.num_pages * kPage);
    CPMCU_CHECK_ARG(q && k_new && v_new && cache_length && out, "decode_attention: null pointer argument");
    hipStream_t st = resolve_stream(nullptr);
    PerfScope perf("DECODE_ATTN_CORE", st);
    // KV append (src/model/attn.cuh:200) is fused into the attention kernel
    const uint64_t* mask = mask_2d ? (const uint64_t*)mask_2d : m.chain_mask;
    return cpmcu_tree_attention((const void*)q, m.k_pools[layer], m.v_pools[layer], m.block_table,
                                (const int32_t*)cache_length, padded_length, (const void*)k_new, (const void*)v_new, mask, 1, 0,
                                input_length, m.q_heads, m.kv_heads, 1.f / sqrtf((float)kHeadDim), (void*)out, m.attn_ws,
                                m.attn_ws_bytes, 0, st);
}

extern "C" int cpmcu_draft_attention(int draft_layer, int input_length, int padded_length, uint64_t q, uint64_t k_new,
                                     uint64_t v_new, uint64_t cache_length, uint64_t mask_2d, int mask_k_range, uint64_t out) {
    int rc = require_model(true);
    if (rc) return rc;
    Model& m = *g_model;
    if (!m.drafter) {
        set_error("draft_attention: no drafter configured");
        return CPMCU_ERR_RUNTIME;
    }
    CPMCU_CHECK_ARG(draft_layer >= 0 && draft_layer < m.draft_layers, "draft_attention: layer %d outside [0, %d)", draft_layer,
                    m.draft_layers);
    CPMCU_CHECK_ARG(input_length >= 1 && input_length <= 64, "draft_attention: input_length=%d outside [1, 64]", input_length);
    CPMCU_CHECK_ARG(padded_length >= input_length && padded_length <= m.num_pages * kPage,
                    "draft_attention: padded_length=%d outside [%d, %d]", padded_length, input_length, m.num_pages * kPage);
    CPMCU_CHECK_ARG(q && k_new && v_new && cache_length && out, "draft_attention: null pointer argument");
    CPMCU_CHECK_ARG(mask_2d ? (mask_k_range >= input_length && mask_k_range <= 64) : mask_k_range == 0,
                    "draft_attention: mask_k_range=%d (one uint64 per row covers [input_length, 64] columns; 0 without a mask)",
                    mask_k_range);
    hipStream_t st = resolve_stream(nullptr);
    PerfScope perf("DRAFT_ATTN_CORE", st);
    const int l = m.layers + draft_layer;
    const uint64_t* mask = mask_2d ? (const uint64_t*)mask_2d : m.chain_mask;
    return cpmcu_tree_attention_window((const void*)q, m.k_pools[l], m.v_pools[l], m.block_table, (const int32_t*)cache_length,
                                       padded_length, (const void*)k_new, (const void*)v_new, nullptr, m.eagle_window, mask, 1,
                                       mask_k_range, input_length, m.q_heads, m.kv_heads, 1.f / sqrtf((float)kHeadDim), (void*)out,
                                       m.attn_ws, m.attn_ws_bytes, 0, st);
}

extern "C" int cpmcu_decode_lm_head(int input_length, uint64_t hidden, uint64_t logits, uint64_t gt) {
    int rc = require_model(true);
    if (rc) return rc;
    Model& m = *g_model;
    CPMCU_CHECK_ARG(m.lm_head_loaded, "decode_lm_head: lm_head.weight has not been loaded");
    hipStream_t st = resolve_stream(nullptr);
    PerfScope perf("DECODE_LM_HEAD", st);
    return cpmcu_lm_head_argmax((const void*)hidden, m.lm_head, CPMCU_W_TILED, input_length, m.vocab, m.hidden, 1, m.scale_lmhead,
                                (void*)logits, (int32_t*)gt, m.head_ws, m.head_ws_bytes, st);
}

extern "C" int cpmcu_draft_head(int n, uint64_t hidden, uint64_t topk_val, uint64_t topk_pos, uint64_t topk_ids) {
    int rc = require_model(true);
    if (rc) return rc;
    Model& m = *g_model;
    if (!m.drafter) {
        set_error("draft_head: no drafter configured");  // src/model/model.cuh:172-173
        return CPMCU_ERR_RUNTIME;
    }
    CPMCU_CHECK_ARG(m.lm_head_loaded, "draft_head: lm_head.weight has not been loaded");
    hipStream_t st = resolve_stream(nullptr);
    PerfScope perf("DRAFT_HEAD", st);
    return cpmcu_frspec_head_topk((const void*)hidden, m.fr_head, CPMCU_W_TILED, m.fr_head != m.lm_head ? m.token_id_remap : nullptr, n,
                                  m.frspec_vocab, m.hidden, m.topk_per_iter, m.draft_logits, m.row_stats,
                                  (void*)topk_val, (int32_t*)topk_pos, (int32_t*)topk_ids, m.head_ws, m.head_ws_bytes, st);
}

// One round of draft() without the drafter's dense layers (src/model/minicpm4/minicpm4_eagle.cuh:319-382): the
// FR-Spec head on the round's hidden rows, log-softmax, top-k and the tree bookkeeping, with the state kept here.
extern "C" int cpmcu_draft_round(int d, uint64_t hidden, uint64_t next_ids, uint64_t parent_rows, uint64_t draft_mask) {
    int rc = require_model(true);
    if (rc) return rc;
    Model& m = *g_model;
    if (!m.drafter) {
        set_error("draft_round: no drafter configured");  // src/model/model.cuh:172-173
        return CPMCU_ERR_RUNTIME;
    }
    CPMCU_CHECK_ARG(m.lm_head_loaded, "draft_round: lm_head.weight has not been loaded");
    CPMCU_CHECK_ARG(d >= 0 && d < m.num_iter, "draft_round: round %d outside [0, %d)", d, m.num_iter);
    CPMCU_CHECK_ARG(d == 0 || d == m.draft_rounds_done, "draft_round: round %d out of order (%d rounds of this draft have run)", d,
                    m.draft_rounds_done);
    CPMCU_CHECK_ARG(hidden && next_ids, "draft_round: null pointer argument");
    hipStream_t st = resolve_stream(nullptr);
    PerfScope perf("DRAFT_ROUND", st);
    const int k = m.topk_per_iter;
    const int n = d == 0 ? 1 : k;  // the last accepted row, then the k rows of the previous round's picks
    const int32_t* remap = m.fr_head != m.lm_head ? m.token_id_remap : nullptr;
    rc = cpmcu_frspec_head_topk((const void*)hidden, m.fr_head, CPMCU_W_TILED, remap, n, m.frspec_vocab, m.hidden, k, m.draft_logits,
                                m.row_stats, m.topk_val, m.topk_pos, m.topk_ids, m.head_ws, m.head_ws_bytes, st);
    if (rc) return rc;
    if (d == 0)
        rc = cpmcu_draft_tree_begin(m.draft_state, k, m.num_iter, m.topk_val, m.topk_pos, remap, (int32_t*)next_ids, (uint64_t*)draft_mask, st);
    else
        rc = cpmcu_draft_tree_extend(m.draft_state, k, m.num_iter, d, m.topk_val, m.topk_pos, remap, (int32_t*)next_ids,
                                     (int32_t*)parent_rows, (uint64_t*)draft_mask, st);
    if (rc) return rc;
    m.draft_rounds_done = d + 1;
    return CPMCU_OK;
}

// The end of draft() (src/model/minicpm4/minicpm4_eagle.cuh:385-393): the tree_size - 1 best candidates of the
// rounds become the tree the verify step consumes.
extern "C" int cpmcu_draft_finish(uint64_t tree_draft_ids, uint64_t tree_position_ids, uint64_t cache_length, uint64_t tree_attn_mask,
                                  uint64_t tree_parent) {
    int rc = require_model(true);
    if (rc) return rc;
    Model& m = *g_model;
    if (!m.drafter) {
        set_error("draft_finish: no drafter configured");
        return CPMCU_ERR_RUNTIME;
    }
    CPMCU_CHECK_ARG(m.draft_rounds_done == m.num_iter, "draft_finish: %d of %d rounds have run", m.draft_rounds_done, m.num_iter);
    CPMCU_CHECK_ARG(tree_draft_ids && tree_position_ids && cache_length && tree_attn_mask && tree_parent, "draft_finish: null pointer argument");
    hipStream_t st = resolve_stream(nullptr);
    PerfScope perf("DRAFT_FINISH", st);
    const int32_t* remap = m.fr_head != m.lm_head ? m.token_id_remap : nullptr;
    rc = cpmcu_draft_tree_finish(m.draft_state, m.topk_per_iter, m.num_iter, m.tree_size, (const int32_t*)cache_length, remap,
                                 (int32_t*)tree_draft_ids, (int32_t*)tree_position_ids, (uint64_t*)tree_attn_mask, (int32_t*)tree_parent, st);
    if (rc) return rc;
    m.draft_rounds_done = 0;
    return CPMCU_OK;
}

extern "C" int cpmcu_verify_and_fix(int num_tokens, uint64_t pred, uint64_t gt, uint64_t position_ids,
                                    uint64_t cache_length, uint64_t attn_mask, uint64_t tree_parent,
                                    int* accept_length) {
    int rc = require_model(true);
    if (rc) return rc;
    Model& m = *g_model;
    if (!m.drafter) {
        set_error("verify is not supported: no drafter configured");  // src/model/model.cuh:172-173
        return CPMCU_ERR_RUNTIME;
    }
    CPMCU_CHECK_ARG(!m.capturing, "verify_and_fix synchronises: it cannot be part of a capture");
    CPMCU_CHECK_ARG(num_tokens >= 1 && num_tokens <= 64, "verify_and_fix: num_tokens=%d outside [1, 64]", num_tokens);
    CPMCU_CHECK_ARG(pred && gt && position_ids && cache_length && attn_mask && tree_parent, "verify_and_fix: null pointer argument");
    hipStream_t st = resolve_stream(nullptr);
    PerfScope perf("VERIFY_AND_FIX", st);
    // One launch accepts and compacts every cache (each workgroup redoes the acceptance, so nothing waits for
    // the accept length); it writes (a, node) straight into pinned host memory, so the single synchronisation
    // of the step (src/model/minicpm4/minicpm4_eagle.cuh:400-401) moves to the end and needs no copy.  The
    // accepted ids replace the draft ids in pred behind it (pred is read by every workgroup of the first launch).
    rc = cpmcu_verify_tail(m.d_k_pools, m.d_v_pools, m.layers, m.block_table, m.kv_heads, num_tokens, (const int32_t*)pred,
                           (const int32_t*)gt, nullptr, 0, 0, (const int32_t*)position_ids, (const int32_t*)cache_length,
                           (const uint64_t*)attn_mask, 1, (const int32_t*)tree_parent, nullptr, 0, nullptr, nullptr, m.d_best, nullptr,
                           m.d_ids, nullptr, m.h_result, st);
    if (rc) return rc;
    rc = cpmcu_verify_tail_inplace(m.d_best, m.d_ids, num_tokens, (int32_t*)pred, nullptr, nullptr, nullptr, 0, st);
    if (rc) return rc;
    rc = synchronize_and_check(st);
    if (accept_length) *accept_length = m.h_result[0];
    return rc;
}

namespace {

struct StepArgs {
    int T, padded_length;
    const uint64_t *q, *k_new, *v_new, *attn_out;  // host arrays [layers] of device addresses
    uint64_t hidden, draft_ids, position_ids, cache_length, kv_length, attn_mask, tree_parent, block_table;
    uint64_t gt_out, accepted_ids, prev_hidden, next_position_ids, result;
    int flags;
};

// Every launch of one verify step, in order, on `st`: per layer the KV append + tree attention on the model's
// paged cache, the target head (arg-max left as partials), the one-launch tail, and with
// CPMCU_COMMIT_ADVANCE_LENGTH the single-workgroup launch that advances the lengths and positions.
int enqueue_verify_step(Model& m, const StepArgs& a, hipStream_t st) {
    const int32_t* table = a.block_table ? (const int32_t*)a.block_table : m.block_table;
    const float scale = 1.f / sqrtf((float)kHeadDim);
    const int mask_words = ceil_div(a.T, 64);  // one uint64 per row up to the reference's 64 nodes, two for wider trees
    for (int l = 0; l < m.layers; ++l) {
        int rc = cpmcu_tree_attention((const void*)a.q[l], m.k_pools[l], m.v_pools[l], table, (const int32_t*)a.kv_length, a.padded_length,
                                      (const void*)a.k_new[l], (const void*)a.v_new[l], (const uint64_t*)a.attn_mask, mask_words, 0, a.T, m.q_heads,
                                      m.kv_heads, scale, (void*)a.attn_out[l], m.attn_ws, m.attn_ws_bytes, 0, st);
        if (rc) return rc;
    }
    int num_partials = 0, stride = 0;
    int rc = cpmcu_lm_head_partials((const void*)a.hidden, m.lm_head, CPMCU_W_TILED, a.T, m.vocab, m.hidden, 1, m.scale_lmhead, nullptr,
                                    m.head_ws, m.head_ws_bytes, &num_partials, &stride, st);
    if (rc) return rc;
    rc = cpmcu_verify_tail(m.d_k_pools, m.d_v_pools, m.layers, table, m.kv_heads, a.T, (const int32_t*)a.draft_ids, nullptr, m.head_ws,
                           num_partials, stride, (const int32_t*)a.position_ids, (const int32_t*)a.cache_length,
                           (const uint64_t*)a.attn_mask, mask_words, (const int32_t*)a.tree_parent, a.prev_hidden ? (const void*)a.hidden : nullptr,
                           m.hidden, (void*)a.prev_hidden, (int32_t*)a.gt_out, m.d_best, nullptr, (int32_t*)a.accepted_ids,
                           (int32_t*)a.next_position_ids, (int32_t*)a.result, st);
    if (rc) return rc;
    if (a.flags & CPMCU_COMMIT_ADVANCE_LENGTH)
        rc = cpmcu_verify_tail_inplace(m.d_best, (const int32_t*)a.accepted_ids, a.T, nullptr, (int32_t*)a.cache_length,
                                       (int32_t*)a.kv_length, (int32_t*)a.position_ids, CPMCU_COMMIT_ADVANCE_LENGTH, st);
    return rc;
}

uint64_t step_signature(const Model& m, const StepArgs& a) {
    uint64_t h = 1469598103934665603ull;
    auto mix = [&](uint64_t v) {
        for (int b = 0; b < 8; ++b) {
            h ^= (v >> (8 * b)) & 0xff;
            h *= 1099511628211ull;
        }
    };
    for (int l = 0; l < m.layers; ++l) {
        mix(a.q[l]);
        mix(a.k_new[l]);
        mix(a.v_new[l]);
        mix(a.attn_out[l]);
    }
    for (uint64_t v : {a.hidden, a.draft_ids, a.position_ids, a.cache_length, a.kv_length, a.attn_mask, a.tree_parent, a.block_table,
                       a.gt_out, a.accepted_ids, a.prev_hidden, a.next_position_ids, a.result, (uint64_t)a.flags})
        mix(v);
    // the options decide which kernels a capture records: a graph captured under other settings is another graph
    const Options& o = options();
    for (int v : {o.dtype, o.attn_kv_groups, o.head_share_last_pass, o.head_stream_kernel, o.attn_merge_in_launch, o.attn_merge_wait_us, o.frspec_fused, o.frspec_wait_us, o.topk_row_kernel}) mix((uint64_t)(uint32_t)v);
    return h;
}


}  // namespace

extern "C" int cpmcu_verify_step(int num_layers, int num_tokens, int padded_length, const uint64_t* q, const uint64_t* k_new, const uint64_t* v_new,
                                 const uint64_t* attn_out, uint64_t hidden, uint64_t draft_ids, uint64_t position_ids,
                                 uint64_t cache_length, uint64_t kv_length, uint64_t attn_mask, uint64_t tree_parent,
                                 uint64_t block_table, uint64_t gt_out, uint64_t accepted_ids, uint64_t prev_hidden,
                                 uint64_t next_position_ids, uint64_t result, int flags, int cuda_graph) {
    int rc = require_model(true);
    if (rc) return rc;
    Model& m = *g_model;
    if (!m.drafter) {
        set_error("verify is not supported: no drafter configured");  // src/model/model.cuh:172-173
        return CPMCU_ERR_RUNTIME;
    }
    CPMCU_CHECK_ARG(m.lm_head_loaded, "verify_step: lm_head.weight has not been loaded");
    CPMCU_CHECK_ARG(num_layers == m.layers, "verify_step: %d per-layer addresses given, the model has %d layers", num_layers, m.layers);
    CPMCU_CHECK_ARG(num_tokens >= 1 && num_tokens <= kMaxTree, "verify_step: num_tokens=%d outside [1, %d]", num_tokens, kMaxTree);
    CPMCU_CHECK_ARG(padded_length >= num_tokens && padded_length <= m.num_pages * kPage, "verify_step: padded_length=%d outside [%d, %d]",
                    padded_length, num_tokens, m.num_pages * kPage);
    CPMCU_CHECK_ARG(q && k_new && v_new && attn_out, "verify_step: null per-layer address array");
    for (int l = 0; l < m.layers; ++l)
        CPMCU_CHECK_ARG(q[l] && k_new[l] && v_new[l] && attn_out[l], "verify_step: null address for layer %d", l);
    CPMCU_CHECK_ARG(hidden && draft_ids && position_ids && cache_length && kv_length && attn_mask && tree_parent && accepted_ids,
                    "verify_step: null pointer argument");
    CPMCU_CHECK_ARG((flags & ~CPMCU_COMMIT_ADVANCE_LENGTH) == 0, "verify_step: unknown flags 0x%x", flags);
    CPMCU_CHECK_ARG(prev_hidden == 0 || prev_hidden != hidden, "verify_step: prev_hidden must not alias hidden (rows are gathered by many workgroups)");
    const StepArgs a{num_tokens, padded_length, q, k_new, v_new, attn_out, hidden, draft_ids, position_ids, cache_length, kv_length,
                     attn_mask, tree_parent, block_table, gt_out, accepted_ids, prev_hidden, next_position_ids, result, flags};
    hipStream_t st = resolve_stream(nullptr);
    if (!cuda_graph) {
        PerfScope perf("VERIFY_STEP", st);
        return enqueue_verify_step(m, a, st);
    }
    CPMCU_CHECK_ARG(!m.capturing, "verify_step: cuda_graph inside an open capture (pass cuda_graph = 0 there)");
    // Graph path, as decode(..., cuda_graph = true) of the reference: captured once per (padded_length, num_tokens)
    // -- and per set of addresses, which a graph bakes in -- and replayed afterwards.  Every length the kernels
    // need is read from device memory, so the same graph serves every step of that padded length.
    const uint64_t sig = step_signature(m, a);
    {
        auto& bucket = m.step_graphs[{padded_length, num_tokens}];
        for (auto& g : bucket)
            if (g.signature == sig) {
                g.last_use = ++m.graph_clock;
                CPMCU_HIP(hipGraphLaunch(g.exec, st));
                return CPMCU_OK;
            }
    }
    // A new graph.  The library keeps at most kMaxStepGraphs of them (the reference keeps one and drops it when the key
    // changes, src/entry.cu:476-484; a caller that rotates over a few sets of buffers or page tables needs a few): the one
    // unused the longest goes first, once the stream has drained -- it may still be running.
    size_t held = 0;
    for (auto& kv : m.step_graphs) held += kv.second.size();
    while (held >= (size_t)kMaxStepGraphs) {
        std::map<std::pair<int, int>, std::vector<Model::StepGraph>>::iterator ob = m.step_graphs.end();
        size_t oi = 0;
        for (auto it = m.step_graphs.begin(); it != m.step_graphs.end(); ++it)
            for (size_t i = 0; i < it->second.size(); ++i)
                if (ob == m.step_graphs.end() || it->second[i].last_use < ob->second[oi].last_use) {
                    ob = it;
                    oi = i;
                }
        CPMCU_HIP(hipStreamSynchronize(st));
        if (ob->second[oi].exec) (void)hipGraphExecDestroy(ob->second[oi].exec);
        if (ob->second[oi].graph) (void)hipGraphDestroy(ob->second[oi].graph);
        ob->second.erase(ob->second.begin() + oi);
        if (ob->second.empty()) m.step_graphs.erase(ob);
        --held;
    }
    Model::StepGraph g;
    g.signature = sig;
    g.last_use = ++m.graph_clock;
    CPMCU_HIP(hipStreamBeginCapture(st, hipStreamCaptureModeRelaxed));
    rc = enqueue_verify_step(m, a, st);
    const hipError_t e = hipStreamEndCapture(st, &g.graph);
    if (rc) {
        if (g.graph) (void)hipGraphDestroy(g.graph);
        return rc;
    }
    if (e != hipSuccess) {
        set_error("verify_step: stream capture failed: %s", hipGetErrorString(e));
        return CPMCU_ERR_HIP;
    }
    {
        const hipError_t ei = hipGraphInstantiate(&g.exec, g.graph, nullptr, nullptr, 0);
        if (ei != hipSuccess) {
            (void)hipGraphDestroy(g.graph);
            set_error("verify_step: hipGraphInstantiate failed: %s", hipGetErrorString(ei));
            return CPMCU_ERR_HIP;
        }
    }
    m.step_graphs[{padded_length, num_tokens}].push_back(g);
    CPMCU_HIP(hipGraphLaunch(g.exec, st));
    return CPMCU_OK;
}

// The same mechanism for any sequence of the model-level calls that only enqueue (decode_attention, draft_attention,
// decode_lm_head, draft_head, draft_round, draft_finish, verify_step without cuda_graph): what is called between
// capture_begin and capture_end is recorded on the library's stream instead of run, and replayed as one graph.
extern "C" int cpmcu_capture_begin(void) {
    int rc = require_model(true);
    if (rc) return rc;
    Model& m = *g_model;
    CPMCU_CHECK_ARG(!m.capturing, "capture_begin: a capture is already open");
    CPMCU_HIP(hipStreamBeginCapture(resolve_stream(nullptr), hipStreamCaptureModeRelaxed));
    m.capturing = true;
    return CPMCU_OK;
}

extern "C" int cpmcu_capture_end(int* graph_id) {
    int rc = require_model(true);
    if (rc) return rc;
    Model& m = *g_model;
    CPMCU_CHECK_ARG(m.capturing, "capture_end: no capture is open");
    CPMCU_CHECK_ARG(graph_id, "capture_end: null pointer argument");
    m.capturing = false;
    Model::StepGraph g;
    const hipError_t e = hipStreamEndCapture(resolve_stream(nullptr), &g.graph);
    if (e != hipSuccess || g.graph == nullptr) {
        set_error("capture_end: stream capture failed: %s", hipGetErrorString(e));
        return CPMCU_ERR_HIP;
    }
    {
        const hipError_t ei = hipGraphInstantiate(&g.exec, g.graph, nullptr, nullptr, 0);
        if (ei != hipSuccess) {
            (void)hipGraphDestroy(g.graph);
            set_error("capture_end: hipGraphInstantiate failed: %s", hipGetErrorString(ei));
            return CPMCU_ERR_HIP;
        }
    }
    // a slot freed by cpmcu_graph_destroy is taken again
    for (size_t i = 0; i < m.user_graphs.size(); ++i)
        if (m.user_graphs[i].exec == nullptr) {
            m.user_graphs[i] = g;
            *graph_id = (int)i;
            return CPMCU_OK;
        }
    m.user_graphs.push_back(g);
    *graph_id = (int)m.user_graphs.size() - 1;
    return CPMCU_OK;
}

extern "C" int cpmcu_graph_destroy(int graph_id) {
    int rc = require_model(true);
    if (rc) return rc;
    Model& m = *g_model;
    CPMCU_CHECK_ARG(graph_id >= 0 && graph_id < (int)m.user_graphs.size() && m.user_graphs[graph_id].exec != nullptr,
                    "graph_destroy: unknown graph %d", graph_id);
    CPMCU_CHECK_ARG(!m.capturing, "graph_destroy: a capture is open");
    CPMCU_HIP(hipStreamSynchronize(resolve_stream(nullptr)));  // it may still be running
    (void)hipGraphExecDestroy(m.user_graphs[graph_id].exec);
    (void)hipGraphDestroy(m.user_graphs[graph_id].graph);
    m.user_graphs[graph_id] = Model::StepGraph{};
    return CPMCU_OK;
}

// Extension for tests and diagnostics: captured verify steps the library holds at the moment.
extern "C" int cpmcu_step_graph_count(void) {
    if (!g_model) return 0;
    int n = 0;
    for (auto& kv : g_model->step_graphs) n += (int)kv.second.size();
    return n;
}

extern "C" int cpmcu_graph_replay(int graph_id) {
    int rc = require_model(true);
    if (rc) return rc;
    Model& m = *g_model;
    CPMCU_CHECK_ARG(graph_id >= 0 && graph_id < (int)m.user_graphs.size() && m.user_graphs[graph_id].exec != nullptr,
                    "graph_replay: unknown graph %d", graph_id);
    CPMCU_CHECK_ARG(!m.capturing, "graph_replay: a capture is open");
    CPMCU_HIP(hipGraphLaunch(m.user_graphs[graph_id].exec, resolve_stream(nullptr)));
    return CPMCU_OK;
}

extern "C" int cpmcu_print_perf_summary(void) {
    if (!g_model) return CPMCU_OK;
    printf("%-24s %10s %12s %12s\n", "label", "count", "total ms", "avg ms");
    for (auto& kv : g_model->perf_log)
        printf("%-24s %10ld %12.3f %12.4f\n", kv.first.c_str(), kv.second.count, kv.second.ms,
               kv.second.count ? kv.second.ms / kv.second.count : 0.0);
    size_t free_b = 0, total_b = 0;
    if (hipMemGetInfo(&free_b, &total_b) == hipSuccess)
        printf("GPU memory: %.1f MiB used of %.1f MiB\n", (total_b - free_b) / 1048576.0, total_b / 1048576.0);
    printf("attention merge waits that ran out (share left to the last workgroup of its unit): %ld\n", g_abandoned_waits);
    printf("one-launch FR-Spec heads: %ld rows from the published candidates, %ld redone from the logits, %ld not finished\n",
           g_frspec_fused_rows, g_frspec_slow_rows, g_frspec_timeouts);
    fflush(stdout);
    return CPMCU_OK;
}

// Extension: merge waits of tree-attention launches that ran out since the library was loaded, as seen by the
// synchronising calls so far (cpmcu_synchronize, cpmcu_verify_and_fix).  Each is a workgroup that stopped waiting for the
// others of its unit and left its share of the merge to the last of them: the output was complete, but late, and the
// device's workspaces have gone back to the separate merge launch (cpmcu_set_option("attn_merge_in_launch", 1) undoes that).
extern "C" long cpmcu_attention_abandoned_waits(void) { return g_abandoned_waits; }

// Rows of one-launch FR-Spec heads seen by the library's synchronisations so far: finished from the published candidates,
// redone from the logits in memory (tie-heavy rows), and not finished because a wait ran out (an error at that
// synchronisation).  Any of the pointers may be null.
extern "C" int cpmcu_frspec_fused_rows(long* fused_rows, long* slow_rows, long* timeouts) {
    if (fused_rows) *fused_rows = g_frspec_fused_rows;
    if (slow_rows) *slow_rows = g_frspec_slow_rows;
    if (timeouts) *timeouts = g_frspec_timeouts;
    return CPMCU_OK;
}

// Extension: device pointers of the model's storage for harnesses that fill the cache directly.
extern "C" int cpmcu_model_pointers(int layer, uint64_t* k_pool, uint64_t* v_pool, uint64_t* block_table,
                                    int* num_pages) {
    int rc = require_model(true);
    if (rc) return rc;
    Model& m = *g_model;
    CPMCU_CHECK_ARG(layer >= 0 && layer < m.layers + m.draft_layers, "model_pointers: layer %d outside [0, %d)", layer,
                    m.layers + m.draft_layers);
    if (k_pool) *k_pool = (uint64_t)m.k_pools[layer];
    if (v_pool) *v_pool = (uint64_t)m.v_pools[layer];
    if (block_table) *block_table = (uint64_t)m.block_table;
    if (num_pages) *num_pages = m.num_pages;
    return CPMCU_OK;
}

extern "C" uint64_t cpmcu_stream(void) { return (uint64_t)(uintptr_t)resolve_stream(nullptr); }

extern "C" int cpmcu_synchronize(void) {
    CPMCU_CHECK_ARG(!(g_model && g_model->capturing), "synchronize: the library's stream is being captured");
    return synchronize_and_check(resolve_stream(nullptr));
}

extern "C" int cpmcu_shutdown(void) {
    if (!g_model) return CPMCU_OK;
    Model& m = *g_model;
    if (g_stream) (void)hipStreamSynchronize(g_stream);
    release_storage(m);
    delete g_model;
    g_model = nullptr;
    options().dtype = 0;  // the operator-level entry points are back on the default element type
    return CPMCU_OK;
}
