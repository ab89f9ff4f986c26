// pybind11 face of the C ABI.  Tensors cross as raw device addresses (torch's data_ptr()) and the
// HIP stream as an integer handle; no torch types appear here.  Argument errors raise ValueError,
// everything else RuntimeError, carrying the library's own message.
#include <pybind11/pybind11.h>
#include <pybind11/stl.h>

#include <stdexcept>
#include <vector>

#include <cstdint>
#include <stdexcept>
#include <string>

#include "pypto_amd_sfa.h"

namespace py = pybind11;

namespace {

void check(int rc)
{
    if (rc == PTO_OK) return;
    const std::string msg = pto_last_error();
    if (rc == PTO_E_INVALID_ARG) throw py::value_error(msg);
    throw std::runtime_error(msg);
}

template <typename T> T *ptr(std::uintptr_t v) { return reinterpret_cast<T *>(v); }

PtoSfaQuantArgs sfa_args(std::uintptr_t query_nope, std::uintptr_t query_rope, std::uintptr_t key_nope_2d,
                         std::uintptr_t key_rope_2d, std::uintptr_t k_nope_scales, std::uintptr_t topk_indices,
                         std::uintptr_t block_table, std::uintptr_t kv_act_seqs, std::uintptr_t attention_out,
                         std::uintptr_t workspace, size_t workspace_bytes, int64_t b, int64_t s1, int64_t nq,
                         int64_t n_kv, int64_t topk, int64_t block_size, int64_t max_blocknum_perbatch,
                         int64_t kv_rows, double softmax_scale, int num_splits)
{
    PtoSfaQuantArgs a{};
    a.query_nope = ptr<const void>(query_nope);
    a.query_rope = ptr<const void>(query_rope);
    a.key_nope_2d = ptr<const void>(key_nope_2d);
    a.key_rope_2d = ptr<const void>(key_rope_2d);
    a.k_nope_scales = ptr<const void>(k_nope_scales);
    a.topk_indices = ptr<const int32_t>(topk_indices);
    a.block_table = ptr<const int32_t>(block_table);
    a.kv_act_seqs = ptr<const int32_t>(kv_act_seqs);
    a.attention_out = ptr<void>(attention_out);
    a.workspace = ptr<void>(workspace);
    a.workspace_bytes = workspace_bytes;
    a.b = b;
    a.s1 = s1;
    a.nq = nq;
    a.n_kv = n_kv;
    a.topk = topk;
    a.block_size = block_size;
    a.max_blocknum_perbatch = max_blocknum_perbatch;
    a.kv_rows = kv_rows;
    a.softmax_scale = static_cast<float>(softmax_scale);
    a.num_splits = num_splits;
    return a;
}

PtoLiDecodeArgs li_args(std::uintptr_t idx_query, std::uintptr_t idx_query_scale, std::uintptr_t idx_key_cache,
                        std::uintptr_t idx_key_scale, std::uintptr_t idx_weight, std::uintptr_t act_seq_key,
                        std::uintptr_t block_table, std::uintptr_t topk_res, std::uintptr_t workspace,
                        size_t workspace_bytes, int64_t t, int64_t b, int64_t n_heads, int64_t head_dim,
                        int64_t block_num, int64_t block_size, int64_t max_blocknum_perbatch, int64_t selected_count,
                        int q_scale_dtype, int k_scale_dtype, int weight_dtype)
{
    PtoLiDecodeArgs a{};
    a.idx_query = ptr<const int8_t>(idx_query);
    a.idx_query_scale = ptr<const void>(idx_query_scale);
    a.idx_key_cache = ptr<const int8_t>(idx_key_cache);
    a.idx_key_scale = ptr<const void>(idx_key_scale);
    a.idx_weight = ptr<const void>(idx_weight);
    a.act_seq_key = ptr<const int32_t>(act_seq_key);
    a.block_table = ptr<const int32_t>(block_table);
    a.topk_res = ptr<int32_t>(topk_res);
    a.workspace = ptr<void>(workspace);
    a.workspace_bytes = workspace_bytes;
    a.t = t;
    a.b = b;
    a.n_heads = n_heads;
    a.head_dim = head_dim;
    a.block_num = block_num;
    a.block_size = block_size;
    a.max_blocknum_perbatch = max_blocknum_perbatch;
    a.selected_count = selected_count;
    a.q_scale_dtype = q_scale_dtype;
    a.k_scale_dtype = k_scale_dtype;
    a.weight_dtype = weight_dtype;
    return a;
}

}  // namespace

PYBIND11_MODULE(_C, m)
{
    m.doc() = "MI355X sparse flash attention + lightning indexer (C ABI: include/pypto_amd_sfa.h)";
    m.attr("DT_FP16") = PTO_DT_FP16;
    m.attr("DT_FP32") = PTO_DT_FP32;
    m.attr("DT_BF16") = PTO_DT_BF16;
    m.def("version", []() { return std::string(pto_version()); });

    m.def("sfa_quant_workspace_bytes",
          [](int64_t b, int64_t s1, int64_t nq, int64_t n_kv, int64_t topk, int64_t block_size,
             int64_t max_blocknum_perbatch, int64_t kv_rows, double softmax_scale, int num_splits) {
              PtoSfaQuantArgs a = sfa_args(0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, b, s1, nq, n_kv, topk, block_size,
                                           max_blocknum_perbatch, kv_rows, softmax_scale, num_splits);
              size_t bytes = 0;
              check(pto_sfa_quant_workspace_bytes(&a, &bytes));
              return bytes;
          });
    m.def("sfa_quant_launch",
          [](std::uintptr_t query_nope, std::uintptr_t query_rope, std::uintptr_t key_nope_2d, std::uintptr_t key_rope_2d,
             std::uintptr_t k_nope_scales, std::uintptr_t topk_indices, std::uintptr_t block_table,
             std::uintptr_t kv_act_seqs, std::uintptr_t attention_out, std::uintptr_t workspace, size_t workspace_bytes,
             int64_t b, int64_t s1, int64_t nq, int64_t n_kv, int64_t topk, int64_t block_size,
             int64_t max_blocknum_perbatch, int64_t kv_rows, double softmax_scale, int num_splits,
             std::uintptr_t stream) {
              PtoSfaQuantArgs a = sfa_args(query_nope, query_rope, key_nope_2d, key_rope_2d, k_nope_scales, topk_indices,
                                           block_table, kv_act_seqs, attention_out, workspace, workspace_bytes, b, s1, nq,
                                           n_kv, topk, block_size, max_blocknum_perbatch, kv_rows, softmax_scale,
                                           num_splits);
              check(pto_sfa_quant_launch(&a, ptr<void>(stream)));
          });

    m.def("sfa_bf16kv_launch",
          [](std::uintptr_t query_nope, std::uintptr_t query_rope, std::uintptr_t key_nope_2d, std::uintptr_t key_rope_2d,
             std::uintptr_t topk_indices, std::uintptr_t block_table, std::uintptr_t kv_act_seqs,
             std::uintptr_t attention_out, std::uintptr_t workspace, size_t workspace_bytes, int64_t b, int64_t s1,
             int64_t nq, int64_t n_kv, int64_t topk, int64_t block_size, int64_t max_blocknum_perbatch, int64_t kv_rows,
             double softmax_scale, int num_splits, std::uintptr_t stream) {
              PtoSfaQuantArgs a = sfa_args(query_nope, query_rope, key_nope_2d, key_rope_2d, 0, topk_indices, block_table,
                                           kv_act_seqs, attention_out, workspace, workspace_bytes, b, s1, nq, n_kv, topk,
                                           block_size, max_blocknum_perbatch, kv_rows, softmax_scale, num_splits);
              check(pto_sfa_bf16kv_launch(&a, ptr<void>(stream)));
          });
    m.def("sa_antiquant_launch",
          [](std::uintptr_t query_nope, std::uintptr_t query_rope, std::uintptr_t nope_cache, std::uintptr_t topk_indices,
             std::uintptr_t block_table, std::uintptr_t kv_act_seqs, std::uintptr_t attention_out, std::uintptr_t workspace,
             size_t workspace_bytes, int64_t b, int64_t s1, int64_t nq, int64_t n_kv, int64_t topk, int64_t block_size,
             int64_t max_blocknum_perbatch, int64_t kv_rows, double softmax_scale, int num_splits, std::uintptr_t stream) {
              PtoSaAntiquantArgs a{};
              a.query_nope = ptr<const void>(query_nope);
              a.query_rope = ptr<const void>(query_rope);
              a.nope_cache = ptr<const void>(nope_cache);
              a.topk_indices = ptr<const int32_t>(topk_indices);
              a.block_table = ptr<const int32_t>(block_table);
              a.kv_act_seqs = ptr<const int32_t>(kv_act_seqs);
              a.attention_out = ptr<void>(attention_out);
              a.workspace = ptr<void>(workspace);
              a.workspace_bytes = workspace_bytes;
              a.b = b;
              a.s1 = s1;
              a.nq = nq;
              a.n_kv = n_kv;
              a.topk = topk;
              a.block_size = block_size;
              a.max_blocknum_perbatch = max_blocknum_perbatch;
              a.kv_rows = kv_rows;
              a.softmax_scale = static_cast<float>(softmax_scale);
              a.num_splits = num_splits;
              check(pto_sa_antiquant_launch(&a, ptr<void>(stream)));
          });

    m.def("li_decode_workspace_bytes",
          [](int64_t t, int64_t b, int64_t n_heads, int64_t head_dim, int64_t block_num, int64_t block_size,
             int64_t max_blocknum_perbatch, int64_t selected_count, int q_dt, int k_dt, int w_dt) {
              PtoLiDecodeArgs a = li_args(0, 0, 0, 0, 0, 0, 0, 0, 0, 0, t, b, n_heads, head_dim, block_num, block_size,
                                          max_blocknum_perbatch, selected_count, q_dt, k_dt, w_dt);
              size_t bytes = 0;
              check(pto_li_decode_workspace_bytes(&a, &bytes));
              return bytes;
          });
    m.def("li_decode_launch",
          [](std::uintptr_t idx_query, std::uintptr_t idx_query_scale, std::uintptr_t idx_key_cache,
             std::uintptr_t idx_key_scale, std::uintptr_t idx_weight, std::uintptr_t act_seq_key,
             std::uintptr_t block_table, std::uintptr_t topk_res, std::uintptr_t workspace, size_t workspace_bytes,
             int64_t t, int64_t b, int64_t n_heads, int64_t head_dim, int64_t block_num, int64_t block_size,
             int64_t max_blocknum_perbatch, int64_t selected_count, int q_dt, int k_dt, int w_dt,
             std::uintptr_t stream, int arith_variant) {
              PtoLiDecodeArgs a = li_args(idx_query, idx_query_scale, idx_key_cache, idx_key_scale, idx_weight, act_seq_key,
                                          block_table, topk_res, workspace, workspace_bytes, t, b, n_heads, head_dim,
                                          block_num, block_size, max_blocknum_perbatch, selected_count, q_dt, k_dt, w_dt);
              a.arith_variant = arith_variant;
              check(pto_li_decode_launch(&a, ptr<void>(stream)));
          },
          py::arg("idx_query"), py::arg("idx_query_scale"), py::arg("idx_key_cache"), py::arg("idx_key_scale"),
          py::arg("idx_weight"), py::arg("act_seq_key"), py::arg("block_table"), py::arg("topk_res"), py::arg("workspace"),
          py::arg("workspace_bytes"), py::arg("t"), py::arg("b"), py::arg("n_heads"), py::arg("head_dim"),
          py::arg("block_num"), py::arg("block_size"), py::arg("max_blocknum_perbatch"), py::arg("selected_count"),
          py::arg("q_dt"), py::arg("k_dt"), py::arg("w_dt"), py::arg("stream"), py::arg("arith_variant") = 0);

    m.def("li_prolog_quant_workspace_bytes", [](int64_t t, int64_t h, int64_t q_lora_rank, int64_t n_heads, int64_t cache_rows) {
        PtoLiPrologQuantArgs a{};
        a.t = t;
        a.h = h;
        a.q_lora_rank = q_lora_rank;
        a.n_heads = n_heads;
        a.cache_rows = cache_rows;
        size_t bytes = 0;
        check(pto_li_prolog_quant_workspace_bytes(&a, &bytes));
        return bytes;
    });
    m.def("li_prolog_quant_launch",
          [](std::uintptr_t x, std::uintptr_t q_norm, std::uintptr_t q_norm_scale, std::uintptr_t w_qb, std::uintptr_t w_qb_scale,
             std::uintptr_t wk, std::uintptr_t w_proj, std::uintptr_t ln_gamma_k, std::uintptr_t ln_beta_k,
             std::uintptr_t cos_idx_rope, std::uintptr_t sin_idx_rope, std::uintptr_t hadamard_q, std::uintptr_t hadamard_k,
             std::uintptr_t k_cache, std::uintptr_t k_cache_scale, std::uintptr_t k_cache_index, std::uintptr_t q_int8,
             std::uintptr_t q_scale, std::uintptr_t weights, std::uintptr_t workspace, size_t workspace_bytes, int64_t t,
             int64_t h, int64_t q_lora_rank, int64_t n_heads, int64_t cache_rows, double eps, int sum_mode, std::uintptr_t stream) {
              PtoLiPrologQuantArgs a{};
              a.sum_mode = sum_mode;
              a.x = ptr<const void>(x);
              a.q_norm = ptr<const int8_t>(q_norm);
              a.q_norm_scale = ptr<const float>(q_norm_scale);
              a.w_qb = ptr<const int8_t>(w_qb);
              a.w_qb_scale = ptr<const float>(w_qb_scale);
              a.wk = ptr<const void>(wk);
              a.w_proj = ptr<const void>(w_proj);
              a.ln_gamma_k = ptr<const void>(ln_gamma_k);
              a.ln_beta_k = ptr<const void>(ln_beta_k);
              a.cos_idx_rope = ptr<const void>(cos_idx_rope);
              a.sin_idx_rope = ptr<const void>(sin_idx_rope);
              a.hadamard_q = ptr<const void>(hadamard_q);
              a.hadamard_k = ptr<const void>(hadamard_k);
              a.k_cache = ptr<int8_t>(k_cache);
              a.k_cache_scale = ptr<void>(k_cache_scale);
              a.k_cache_index = ptr<const int64_t>(k_cache_index);
              a.q_int8 = ptr<int8_t>(q_int8);
              a.q_scale = ptr<void>(q_scale);
              a.weights = ptr<void>(weights);
              a.workspace = ptr<void>(workspace);
              a.workspace_bytes = workspace_bytes;
              a.t = t;
              a.h = h;
              a.q_lora_rank = q_lora_rank;
              a.n_heads = n_heads;
              a.cache_rows = cache_rows;
              a.eps = static_cast<float>(eps);
              check(pto_li_prolog_quant_launch(&a, ptr<void>(stream)));
          });

    m.def("mla_prolog_quant_workspace_bytes", [](int64_t t, int64_t h, int64_t q_lora_rank, int64_t n_heads, int64_t cache_rows) {
        PtoMlaPrologQuantArgs a{};
        a.t = t;
        a.h = h;
        a.q_lora_rank = q_lora_rank;
        a.n_heads = n_heads;
        a.cache_rows = cache_rows;
        size_t bytes = 0;
        check(pto_mla_prolog_quant_workspace_bytes(&a, &bytes));
        return bytes;
    });
    m.def("mla_prolog_quant_launch",
          [](std::uintptr_t token_x, std::uintptr_t w_dq, std::uintptr_t w_uq_qr, std::uintptr_t dequant_scale, std::uintptr_t w_uk,
             std::uintptr_t w_dkv_kr, std::uintptr_t gamma_cq, std::uintptr_t gamma_ckv, std::uintptr_t cos, std::uintptr_t sin,
             std::uintptr_t cache_index, std::uintptr_t kv_cache, std::uintptr_t kr_cache, std::uintptr_t k_scale_cache,
             std::uintptr_t q_norm_out, std::uintptr_t q_norm_scale_out, std::uintptr_t query_nope_out,
             std::uintptr_t query_rope_out, std::uintptr_t workspace, size_t workspace_bytes, int64_t t, int64_t h,
             int64_t q_lora_rank, int64_t n_heads, int64_t cache_rows, double epsilon_cq, double epsilon_ckv,
             bool absorb_exact, std::uintptr_t stream) {
              PtoMlaPrologQuantArgs a{};
              a.token_x = ptr<const void>(token_x);
              a.w_dq = ptr<const void>(w_dq);
              a.w_uq_qr = ptr<const int8_t>(w_uq_qr);
              a.dequant_scale = ptr<const float>(dequant_scale);
              a.w_uk = ptr<const void>(w_uk);
              a.w_dkv_kr = ptr<const void>(w_dkv_kr);
              a.gamma_cq = ptr<const void>(gamma_cq);
              a.gamma_ckv = ptr<const void>(gamma_ckv);
              a.cos = ptr<const void>(cos);
              a.sin = ptr<const void>(sin);
              a.cache_index = ptr<const int64_t>(cache_index);
              a.kv_cache = ptr<int8_t>(kv_cache);
              a.kr_cache = ptr<void>(kr_cache);
              a.k_scale_cache = ptr<float>(k_scale_cache);
              a.q_norm_out = ptr<int8_t>(q_norm_out);
              a.q_norm_scale_out = ptr<float>(q_norm_scale_out);
              a.query_nope_out = ptr<void>(query_nope_out);
              a.query_rope_out = ptr<void>(query_rope_out);
              a.workspace = ptr<void>(workspace);
              a.workspace_bytes = workspace_bytes;
              a.t = t;
              a.h = h;
              a.q_lora_rank = q_lora_rank;
              a.n_heads = n_heads;
              a.cache_rows = cache_rows;
              a.epsilon_cq = static_cast<float>(epsilon_cq);
              a.epsilon_ckv = static_cast<float>(epsilon_ckv);
              a.absorb_exact = absorb_exact ? 1 : 0;
              check(pto_mla_prolog_quant_launch(&a, ptr<void>(stream)));
          });

    // both prologs as one operator: the pointers of each half in the order of its own launch function
    // (18 of the MLA prolog up to query_rope_out, 19 of the indexer prolog up to weights; the ones the
    // fused entry point ignores may be 0)
    auto fused_args = [](const std::vector<std::uintptr_t> &m, const std::vector<std::uintptr_t> &x, std::uintptr_t workspace,
                         size_t workspace_bytes, int64_t t, int64_t h, int64_t q_lora_rank, int64_t mla_heads,
                         int64_t mla_cache_rows, double epsilon_cq, double epsilon_ckv, bool absorb_exact, int64_t idx_heads,
                         int64_t idx_cache_rows, double idx_eps, int idx_sum_mode) {
        if (m.size() != 18 || x.size() != 19) throw std::invalid_argument("mla_indexer_prolog: 18 + 19 pointers expected");
        PtoMlaIndexerPrologQuantArgs a{};
        a.mla.token_x = ptr<const void>(m[0]);
        a.mla.w_dq = ptr<const void>(m[1]);
        a.mla.w_uq_qr = ptr<const int8_t>(m[2]);
        a.mla.dequant_scale = ptr<const float>(m[3]);
        a.mla.w_uk = ptr<const void>(m[4]);
        a.mla.w_dkv_kr = ptr<const void>(m[5]);
        a.mla.gamma_cq = ptr<const void>(m[6]);
        a.mla.gamma_ckv = ptr<const void>(m[7]);
        a.mla.cos = ptr<const void>(m[8]);
        a.mla.sin = ptr<const void>(m[9]);
        a.mla.cache_index = ptr<const int64_t>(m[10]);
        a.mla.kv_cache = ptr<int8_t>(m[11]);
        a.mla.kr_cache = ptr<void>(m[12]);
        a.mla.k_scale_cache = ptr<float>(m[13]);
        a.mla.q_norm_out = ptr<int8_t>(m[14]);
        a.mla.q_norm_scale_out = ptr<float>(m[15]);
        a.mla.query_nope_out = ptr<void>(m[16]);
        a.mla.query_rope_out = ptr<void>(m[17]);
        a.mla.t = t;
        a.mla.h = h;
        a.mla.q_lora_rank = q_lora_rank;
        a.mla.n_heads = mla_heads;
        a.mla.cache_rows = mla_cache_rows;
        a.mla.epsilon_cq = static_cast<float>(epsilon_cq);
        a.mla.epsilon_ckv = static_cast<float>(epsilon_ckv);
        a.mla.absorb_exact = absorb_exact ? 1 : 0;
        a.indexer.w_qb = ptr<const int8_t>(x[3]);
        a.indexer.w_qb_scale = ptr<const float>(x[4]);
        a.indexer.wk = ptr<const void>(x[5]);
        a.indexer.w_proj = ptr<const void>(x[6]);
        a.indexer.ln_gamma_k = ptr<const void>(x[7]);
        a.indexer.ln_beta_k = ptr<const void>(x[8]);
        a.indexer.hadamard_q = ptr<const void>(x[11]);
        a.indexer.hadamard_k = ptr<const void>(x[12]);
        a.indexer.k_cache = ptr<int8_t>(x[13]);
        a.indexer.k_cache_scale = ptr<void>(x[14]);
        a.indexer.q_int8 = ptr<int8_t>(x[16]);
        a.indexer.q_scale = ptr<void>(x[17]);
        a.indexer.weights = ptr<void>(x[18]);
        a.indexer.n_heads = idx_heads;
        a.indexer.cache_rows = idx_cache_rows;
        a.indexer.eps = static_cast<float>(idx_eps);
        a.indexer.sum_mode = idx_sum_mode;
        a.workspace = ptr<void>(workspace);
        a.workspace_bytes = workspace_bytes;
        return a;
    };
    m.def("mla_indexer_prolog_quant_workspace_bytes",
          [fused_args](int64_t t, int64_t h, int64_t q_lora_rank, int64_t mla_heads, int64_t mla_cache_rows, int64_t idx_heads,
                       int64_t idx_cache_rows) {
              const std::vector<std::uintptr_t> m18(18, 0), x19(19, 0);
              PtoMlaIndexerPrologQuantArgs a = fused_args(m18, x19, 0, 0, t, h, q_lora_rank, mla_heads, mla_cache_rows, 0.0, 0.0,
                                                          false, idx_heads, idx_cache_rows, 0.0, 0);
              size_t bytes = 0;
              check(pto_mla_indexer_prolog_quant_workspace_bytes(&a, &bytes));
              return bytes;
          });
    m.def("mla_indexer_prolog_quant_launch",
          [fused_args](const std::vector<std::uintptr_t> &mla_ptrs, const std::vector<std::uintptr_t> &idx_ptrs,
                       std::uintptr_t workspace, size_t workspace_bytes, int64_t t, int64_t h, int64_t q_lora_rank,
                       int64_t mla_heads, int64_t mla_cache_rows, double epsilon_cq, double epsilon_ckv, bool absorb_exact,
                       int64_t idx_heads, int64_t idx_cache_rows, double idx_eps, int idx_sum_mode, std::uintptr_t stream) {
              PtoMlaIndexerPrologQuantArgs a = fused_args(mla_ptrs, idx_ptrs, workspace, workspace_bytes, t, h, q_lora_rank,
                                                          mla_heads, mla_cache_rows, epsilon_cq, epsilon_ckv, absorb_exact,
                                                          idx_heads, idx_cache_rows, idx_eps, idx_sum_mode);
              check(pto_mla_indexer_prolog_quant_launch(&a, ptr<void>(stream)));
          });
}
