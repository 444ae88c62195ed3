// pybind11 module `C`: the function names and positional signatures of the reference's pybind
// module (src/entry.cu:510-534) over the C-ABI of libcpmcu_amd.  Pointers are raw addresses
// (tensor.data_ptr()) exactly as there.  No torch types, no HIP calls: this file is plain C++.
#include <pybind11/pybind11.h>
#include <pybind11/stl.h>

#include <cstdint>
#include <stdexcept>
#include <string>
#include <vector>

#include "cpmcu_amd.h"

namespace py = pybind11;

namespace {

// std::invalid_argument -> ValueError and std::runtime_error -> RuntimeError, as exceptions cross
// pybind in the reference (src/model/model.cuh:131-135,172-173; src/entry.cu:43,52).
void check(int rc) {
    if (rc == CPMCU_OK) return;
    const std::string msg = cpmcu_last_error();
    if (rc == CPMCU_ERR_INVALID_ARGUMENT) throw py::value_error(msg);
    throw std::runtime_error(msg);
}

[[noreturn]] void out_of_scope(const char* name) {
    throw std::runtime_error(std::string(name) +
                             " builds a model variant (sparse attention / W4A16 / hierarchical drafter) that is "
                             "outside the verify/draft path of this library");
}

}  // namespace

PYBIND11_MODULE(C, m) {
    m.doc() = "MI355X implementation of CPM.cu's speculative-decoding verify/draft path (entry points of src/entry.cu)";

    // base bind -- src/entry.cu:100-136
    m.def("init_base_model",
          [](float memory_limit, int vocab_size, int num_hidden_layers, int hidden_size, int intermediate_size,
             int num_attention_heads, int num_key_value_heads, int head_dim, float rms_norm_eps, int torch_dtype,
             int chunk_length, float scale_embed, float scale_lmhead, float scale_residual) {
              check(cpmcu_init_base_model(memory_limit, vocab_size, num_hidden_layers, hidden_size, intermediate_size,
                                          num_attention_heads, num_key_value_heads, head_dim, rms_norm_eps, torch_dtype,
                                          chunk_length, scale_embed, scale_lmhead, scale_residual));
          },
          "Init base model");
    // model variants outside the path -- src/entry.cu:138-276,343-459
    m.def("init_minicpm4_model", [](py::args) { out_of_scope("init_minicpm4_model"); }, "Init minicpm4 model");
    m.def("init_w4a16_gptq_marlin_base_model", [](py::args) { out_of_scope("init_w4a16_gptq_marlin_base_model"); }, "Init W4A16 base model");
    m.def("init_w4a16_gptq_marlin_minicpm4_model", [](py::args) { out_of_scope("init_w4a16_gptq_marlin_minicpm4_model"); }, "Init W4A16 base model");
    m.def("init_w4a16_gm_spec_w4a16_gm_model", [](py::args) { out_of_scope("init_w4a16_gm_spec_w4a16_gm_model"); }, "Init w4a16 spec v1 model");
    m.def("init_hier_eagle_w4a16_gm_spec_w4a16_gm_model", [](py::args) { out_of_scope("init_hier_eagle_w4a16_gm_spec_w4a16_gm_model"); }, "init hier eagle gm spec gm model");
    m.def("init_hier_eagle_w4a16_gm_rot_spec_w4a16_gm_model", [](py::args) { out_of_scope("init_hier_eagle_w4a16_gm_rot_spec_w4a16_gm_model"); }, "init hier eagle rot gm spec gm model");

    // eagle bind -- src/entry.cu:278-341
    m.def("init_eagle_model",
          [](int num_layers, int num_iter, int topk_per_iter, int tree_size, int torch_dtype) {
              check(cpmcu_init_eagle_model(num_layers, num_iter, topk_per_iter, tree_size, torch_dtype));
          },
          "Init eagle model");
    m.def("init_minicpm4_eagle_model",
          [](int num_layers, int num_iter, int topk_per_iter, int tree_size, int torch_dtype, bool apply_eagle_quant,
             int group_size, int eagle_window_size, int frspec_vocab_size, float residual_scale, bool use_input_norm,
             bool use_attn_norm) {
              check(cpmcu_init_minicpm4_eagle_model(num_layers, num_iter, topk_per_iter, tree_size, torch_dtype,
                                                    apply_eagle_quant, group_size, eagle_window_size, frspec_vocab_size,
                                                    residual_scale, use_input_norm, use_attn_norm));
          },
          "Init minicpm4 eagle model");

    // interface -- src/entry.cu:462-508
    m.def("init_storage",
          []() {
              int max_context = 0;
              check(cpmcu_init_storage(&max_context));
              return max_context;
          },
          "Init storage");
    m.def("load_model", [](std::string name, std::uintptr_t param) { check(cpmcu_load_model(name.c_str(), (uint64_t)param)); }, "Load model");
    m.def("prefill",
          [](int input_length, int history_length, std::uintptr_t input, std::uintptr_t position_ids, std::uintptr_t output) {
              check(cpmcu_prefill(input_length, history_length, input, position_ids, output));
          },
          "Prefill");
    m.def("decode",
          [](int input_length, int padded_length, std::uintptr_t input, std::uintptr_t position_ids, std::uintptr_t cache_length,
             std::uintptr_t mask_2d, std::uintptr_t output, bool cuda_graph) {
              check(cpmcu_decode(input_length, padded_length, input, position_ids, cache_length, mask_2d, output, cuda_graph));
          },
          "Decode");
    m.def("draft",
          [](std::uintptr_t tree_draft_ids, std::uintptr_t tree_position_ids, std::uintptr_t cache_length, std::uintptr_t attn_mask,
             std::uintptr_t tree_parent) { check(cpmcu_draft(tree_draft_ids, tree_position_ids, cache_length, attn_mask, tree_parent)); },
          "Draft");
    m.def("verify_and_fix",
          [](int num_tokens, std::uintptr_t pred, std::uintptr_t gt, std::uintptr_t position_ids, std::uintptr_t cache_length,
             std::uintptr_t attn_mask, std::uintptr_t tree_parent) {
              int accept = 0;
              check(cpmcu_verify_and_fix(num_tokens, pred, gt, position_ids, cache_length, attn_mask, tree_parent, &accept));
              return accept;
          },
          "Verify and fix");
    m.def("print_perf_summary", []() { check(cpmcu_print_perf_summary()); }, "Print perf summary");

    // the parts of decode / draft that are on the path (no counterpart in the reference's module)
    m.def("decode_attention",
          [](int layer, int input_length, int padded_length, std::uintptr_t q, std::uintptr_t k_new, std::uintptr_t v_new,
             std::uintptr_t cache_length, std::uintptr_t mask_2d, std::uintptr_t out) {
              check(cpmcu_decode_attention(layer, input_length, padded_length, q, k_new, v_new, cache_length, mask_2d, out));
          },
          "KV append + tree attention of one layer on the model's paged cache");
    m.def("draft_attention",
          [](int draft_layer, int input_length, int padded_length, std::uintptr_t q, std::uintptr_t k_new, std::uintptr_t v_new,
             std::uintptr_t cache_length, std::uintptr_t mask_2d, int mask_k_range, std::uintptr_t out) {
              check(cpmcu_draft_attention(draft_layer, input_length, padded_length, q, k_new, v_new, cache_length, mask_2d,
                                          mask_k_range, out));
          },
          "KV append + windowed attention of one of the drafter's own layers on its paged cache");
    m.def("decode_lm_head",
          [](int input_length, std::uintptr_t hidden, std::uintptr_t logits, std::uintptr_t gt) {
              check(cpmcu_decode_lm_head(input_length, hidden, logits, gt));
          },
          "Target lm_head with fused arg-max");
    m.def("draft_head",
          [](int n, std::uintptr_t hidden, std::uintptr_t topk_val, std::uintptr_t topk_pos, std::uintptr_t topk_ids) {
              check(cpmcu_draft_head(n, hidden, topk_val, topk_pos, topk_ids));
          },
          "FR-Spec draft head + log-softmax + top-k + id map-back");
    m.def("draft_round",
          [](int d, std::uintptr_t hidden, std::uintptr_t next_ids, std::uintptr_t parent_rows, std::uintptr_t draft_mask) {
              check(cpmcu_draft_round(d, hidden, next_ids, parent_rows, draft_mask));
          },
          "One round of draft() without the drafter's dense layers: FR-Spec head + log-softmax + top-k + tree bookkeeping");
    m.def("draft_finish",
          [](std::uintptr_t tree_draft_ids, std::uintptr_t tree_position_ids, std::uintptr_t cache_length, std::uintptr_t attn_mask,
             std::uintptr_t tree_parent) { check(cpmcu_draft_finish(tree_draft_ids, tree_position_ids, cache_length, attn_mask, tree_parent)); },
          "The end of draft(): the final selection and the tree the verify step consumes");
    m.def("verify_step",
          [](int num_tokens, int padded_length, std::vector<std::uintptr_t> q, std::vector<std::uintptr_t> k_new,
             std::vector<std::uintptr_t> v_new, std::vector<std::uintptr_t> attn_out, std::uintptr_t hidden, std::uintptr_t draft_ids,
             std::uintptr_t position_ids, std::uintptr_t cache_length, std::uintptr_t kv_length, std::uintptr_t attn_mask,
             std::uintptr_t tree_parent, std::uintptr_t block_table, std::uintptr_t gt_out, std::uintptr_t accepted_ids,
             std::uintptr_t prev_hidden, std::uintptr_t next_position_ids, std::uintptr_t result, int flags, bool cuda_graph) {
              if (q.size() != k_new.size() || q.size() != v_new.size() || q.size() != attn_out.size())
                  throw py::value_error("verify_step: the per-layer address lists differ in length");
              std::vector<uint64_t> a(q.begin(), q.end()), b(k_new.begin(), k_new.end()), c(v_new.begin(), v_new.end()),
                  d(attn_out.begin(), attn_out.end());
              check(cpmcu_verify_step((int)a.size(), num_tokens, padded_length, a.data(), b.data(), c.data(), d.data(), hidden, draft_ids,
                                              position_ids, cache_length, kv_length, attn_mask, tree_parent, block_table, gt_out,
                                              accepted_ids, prev_hidden, next_position_ids, result, flags, cuda_graph));
          },
          "One verify step of the path (attention of every layer, target head, acceptance, compaction), optionally as a replayed graph");
    m.def("synchronize", []() { check(cpmcu_synchronize()); });
    m.def("shutdown", []() { check(cpmcu_shutdown()); });
}
