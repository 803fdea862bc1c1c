// torch.library bindings for the vllm_amd CDNA4 kernels.
//
// Loaded via torch.ops.load_library("vllm_amd/_C.so"); ops appear as
// torch.ops.vllm_amd.<name>. No Python C API — pure libtorch, same
// pattern as the reference's csrc/libtorch_stable/torch_bindings.cpp.

#include <torch/all.h>
#include <torch/library.h>

namespace vllm_amd {

torch::Tensor rms_norm(torch::Tensor x, torch::Tensor weight, double eps);
void fused_add_rms_norm(torch::Tensor x, torch::Tensor residual,
                        torch::Tensor weight, double eps);
torch::Tensor silu_and_mul(torch::Tensor x);
torch::Tensor gelu_and_mul(torch::Tensor x);
void rotary_embedding(torch::Tensor positions, torch::Tensor q,
                      torch::Tensor k, torch::Tensor cos_sin_cache,
                      int64_t rot);
void reshape_and_cache(torch::Tensor key, torch::Tensor value,
                       torch::Tensor kv_cache, torch::Tensor slot_mapping);
void paged_decode_attention(torch::Tensor out, torch::Tensor q,
                            torch::Tensor kv_cache,
                            torch::Tensor block_table,
                            torch::Tensor seq_lens, double scale,
                            int64_t max_seq_len, int64_t sliding_window,
                            torch::Tensor tmp_out, torch::Tensor tmp_lse);
void prefill_attention(torch::Tensor out, torch::Tensor q,
                       torch::Tensor kv_cache, torch::Tensor block_table,
                       torch::Tensor query_start_loc, torch::Tensor seq_lens,
                       double scale, int64_t num_decodes,
                       int64_t max_query_len, int64_t sliding_window);
torch::Tensor lt_linear(torch::Tensor a, torch::Tensor w,
                        c10::optional<torch::Tensor> bias);
torch::Tensor lt_linear_fp8(torch::Tensor a, torch::Tensor w);
void dynamic_quant_fp8(torch::Tensor out, torch::Tensor scales,
                       torch::Tensor x);
void scale_rows_cols(torch::Tensor y, torch::Tensor row_scales,
                     torch::Tensor col_scales,
                     c10::optional<torch::Tensor> bias);
void moe_align(torch::Tensor topk_ids, int64_t num_experts,
               torch::Tensor sorted, torch::Tensor expert_tiles,
               torch::Tensor inv_perm, torch::Tensor counts,
               torch::Tensor fill, torch::Tensor off);
void moe_gemm(torch::Tensor a, torch::Tensor b, torch::Tensor c,
              torch::Tensor sorted, torch::Tensor expert_tiles,
              int64_t topk_div, int64_t total_flat);
void moe_combine(torch::Tensor out, torch::Tensor y,
                 torch::Tensor topk_weights, torch::Tensor inv_perm);
void moe_gemm_shuf(torch::Tensor a, torch::Tensor b_shuf, torch::Tensor c,
                   torch::Tensor sorted, torch::Tensor expert_tiles,
                   int64_t n, int64_t k, int64_t topk_div,
                   int64_t total_flat);
void mla_decode(torch::Tensor out, torch::Tensor q_nope, torch::Tensor q_pe,
                torch::Tensor kv_cache, torch::Tensor block_table,
                torch::Tensor seq_lens, double scale, int64_t max_seq_len,
                torch::Tensor tmp_out, torch::Tensor tmp_lse);
torch::Tensor scalar_rms_norm(torch::Tensor x, torch::Tensor gain,
                              double eps, torch::ScalarType out_dtype);
torch::Tensor add_scaled_scalar_norm(
    torch::Tensor residual, torch::Tensor y, torch::Tensor gain, double eps,
    double mult, c10::optional<torch::ScalarType> out_dtype);
torch::Tensor token_shift(torch::Tensor x, torch::Tensor mu,
                          c10::optional<torch::Tensor> state,
                          c10::optional<torch::Tensor> state_rows,
                          torch::Tensor query_start_loc,
                          torch::ScalarType out_dtype);
torch::Tensor silu_and_mul_any(torch::Tensor x);
torch::Tensor norm_qk_cache_write(torch::Tensor q, torch::Tensor k,
                                  torch::Tensor v,
                                  c10::optional<torch::Tensor> q_w,
                                  c10::optional<torch::Tensor> k_w, double eps,
                                  torch::Tensor k_cache, torch::Tensor v_cache,
                                  torch::Tensor slot_mapping);
void pool_update(torch::Tensor k_cache, torch::Tensor v_cache,
                 torch::Tensor pool_k, torch::Tensor pool_v,
                 torch::Tensor block_table, torch::Tensor query_start_loc,
                 torch::Tensor seq_lens, int64_t pool, int64_t max_query_len);
void pooled_window_attention_rows(
    torch::Tensor out, torch::Tensor q, torch::Tensor k_cache,
    torch::Tensor v_cache, torch::Tensor pool_k, torch::Tensor pool_v,
    torch::Tensor block_table, torch::Tensor query_start_loc,
    torch::Tensor seq_lens, c10::optional<torch::Tensor> gate, double scale,
    int64_t window, int64_t pool, int64_t row0, int64_t num_rows);
void pooled_window_attention_prefill(
    torch::Tensor out, torch::Tensor q, torch::Tensor k_cache,
    torch::Tensor v_cache, torch::Tensor pool_k, torch::Tensor pool_v,
    torch::Tensor block_table, torch::Tensor query_start_loc,
    torch::Tensor seq_lens, c10::optional<torch::Tensor> gate, double scale,
    int64_t window, int64_t pool, int64_t num_decodes,
    int64_t max_query_len);
void pooled_window_attention_decode(
    torch::Tensor out, torch::Tensor q, torch::Tensor k_cache,
    torch::Tensor v_cache, torch::Tensor pool_k, torch::Tensor pool_v,
    torch::Tensor block_table, torch::Tensor query_start_loc,
    torch::Tensor seq_lens, c10::optional<torch::Tensor> gate, double scale,
    int64_t window, int64_t pool, int64_t num_decodes, int64_t max_seq_len);
torch::Tensor scaled_embedding(torch::Tensor ids, torch::Tensor table,
                               double scale);
torch::Tensor rms_norm_cast(torch::Tensor x, torch::Tensor weight,
                            double eps, torch::ScalarType out_dtype);
torch::Tensor add_rms_norm(torch::Tensor residual, torch::Tensor y,
                           torch::Tensor weight, double eps,
                           c10::optional<torch::ScalarType> out_dtype);
torch::Tensor relu2(torch::Tensor x);
torch::Tensor logit_softcap(torch::Tensor logits, double cap);
torch::Tensor sigmoid_gate_mul(torch::Tensor x, torch::Tensor gate);
void latent_rope_cache_write(torch::Tensor q,
                             c10::optional<torch::Tensor> dkv,
                             c10::optional<torch::Tensor> norm_w, double eps,
                             torch::Tensor positions, torch::Tensor inv_freq,
                             int64_t nope_dim, int64_t kv_rank,
                             c10::optional<torch::Tensor> cache,
                             c10::optional<torch::Tensor> slot_mapping);
void latent_attention_rows(torch::Tensor out, torch::Tensor q_abs,
                           torch::Tensor q_rot, torch::Tensor cache,
                           torch::Tensor block_table,
                           torch::Tensor query_start_loc,
                           torch::Tensor seq_lens,
                           c10::optional<torch::Tensor> sink, double scale);
bool latent_attention_tiles_supported(int64_t kv_rank, int64_t rot_dim);
void latent_attention_tiles(torch::Tensor out, torch::Tensor q_abs,
                            torch::Tensor q_rot, torch::Tensor cache,
                            torch::Tensor block_table,
                            torch::Tensor query_start_loc,
                            torch::Tensor seq_lens,
                            c10::optional<torch::Tensor> sink, double scale,
                            int64_t num_decodes, int64_t max_seq_len);
torch::Tensor causal_conv_silu(torch::Tensor x, torch::Tensor weight,
                               torch::Tensor bias,
                               c10::optional<torch::Tensor> conv_state,
                               c10::optional<torch::Tensor> state_rows,
                               torch::Tensor query_start_loc,
                               torch::ScalarType out_dtype);
torch::Tensor ssd_scan(torch::Tensor xbc, int64_t heads, int64_t head_dim,
                       int64_t groups, int64_t state, torch::Tensor dt,
                       torch::Tensor dt_bias, torch::Tensor a_log,
                       torch::Tensor d_skip,
                       c10::optional<torch::Tensor> ssm_state,
                       c10::optional<torch::Tensor> state_rows,
                       torch::Tensor query_start_loc,
                       int64_t max_query_len);
torch::Tensor gated_group_rms_norm(torch::Tensor y, torch::Tensor z,
                                   torch::Tensor weight, double eps,
                                   int64_t groups,
                                   torch::ScalarType out_dtype);
torch::Tensor car_init(int64_t rank, int64_t world, int64_t max_bytes);
void car_connect(torch::Tensor handles);
bool car_is_ready();
int64_t car_max_bytes();
int64_t car_error();
void car_destroy();
void car_all_reduce(torch::Tensor t);
void car_all_gather(torch::Tensor out, torch::Tensor t);
void car_reduce_scatter(torch::Tensor out, torch::Tensor t);

}  // namespace vllm_amd

TORCH_LIBRARY(vllm_amd, m) {
  m.def("rms_norm(Tensor x, Tensor weight, float eps) -> Tensor");
  m.def("fused_add_rms_norm(Tensor(a!) x, Tensor(b!) residual, "
        "Tensor weight, float eps) -> ()");
  m.def("silu_and_mul(Tensor x) -> Tensor");
  m.def("gelu_and_mul(Tensor x) -> Tensor");
  m.def("rotary_embedding(Tensor positions, Tensor(a!) q, Tensor(b!) k, "
        "Tensor cos_sin_cache, int rot) -> ()");
  m.def("reshape_and_cache(Tensor key, Tensor value, Tensor(a!) kv_cache, "
        "Tensor slot_mapping) -> ()");
  m.def("paged_decode_attention(Tensor(a!) out, Tensor q, Tensor kv_cache, "
        "Tensor block_table, Tensor seq_lens, float scale, int max_seq_len, "
        "int sliding_window, Tensor(b!) tmp_out, Tensor(c!) tmp_lse) -> ()");
  m.def("prefill_attention(Tensor(a!) out, Tensor q, Tensor kv_cache, "
        "Tensor block_table, Tensor query_start_loc, Tensor seq_lens, "
        "float scale, int num_decodes, int max_query_len, "
        "int sliding_window) -> ()");
  m.def("lt_linear(Tensor a, Tensor w, Tensor? bias) -> Tensor");
  m.def("lt_linear_fp8(Tensor a, Tensor w) -> Tensor");
  m.def("dynamic_quant_fp8(Tensor(a!) out, Tensor(b!) scales, Tensor x)"
        " -> ()");
  m.def("scale_rows_cols(Tensor(a!) y, Tensor row_scales, Tensor col_scales,"
        " Tensor? bias) -> ()");
  m.def("moe_align(Tensor topk_ids, int num_experts, Tensor(a!) sorted, "
        "Tensor(b!) expert_tiles, Tensor(c!) inv_perm, Tensor(d!) counts, "
        "Tensor(e!) fill, Tensor(f!) off) -> ()");
  m.def("moe_gemm(Tensor a, Tensor b, Tensor(a!) c, Tensor sorted, "
        "Tensor expert_tiles, int topk_div, int total_flat) -> ()");
  m.def("moe_combine(Tensor(a!) out, Tensor y, Tensor topk_weights, "
        "Tensor inv_perm) -> ()");
  m.def("moe_gemm_shuf(Tensor a, Tensor b_shuf, Tensor(a!) c, "
        "Tensor sorted, Tensor expert_tiles, int n, int k, int topk_div, "
        "int total_flat) -> ()");
  m.def("mla_decode(Tensor(a!) out, Tensor q_nope, Tensor q_pe, "
        "Tensor kv_cache, Tensor block_table, Tensor seq_lens, "
        "float scale, int max_seq_len, Tensor(b!) tmp_out, "
        "Tensor(c!) tmp_lse) -> ()");
  m.def("scalar_rms_norm(Tensor x, Tensor gain, float eps, "
        "ScalarType out_dtype) -> Tensor");
  m.def("add_scaled_scalar_norm(Tensor(a!) residual, Tensor y, Tensor gain, "
        "float eps, float mult, ScalarType? out_dtype) -> Tensor");
  m.def("token_shift(Tensor x, Tensor mu, Tensor(a!)? state, "
        "Tensor? state_rows, Tensor query_start_loc, ScalarType out_dtype)"
        " -> Tensor");
  m.def("silu_and_mul_any(Tensor x) -> Tensor");
  m.def("norm_qk_cache_write(Tensor q, Tensor k, Tensor v, Tensor? q_w, "
        "Tensor? k_w, float eps, Tensor(a!) k_cache, Tensor(b!) v_cache, "
        "Tensor slot_mapping) -> Tensor");
  m.def("pool_update(Tensor k_cache, Tensor v_cache, Tensor(a!) pool_k, "
        "Tensor(b!) pool_v, Tensor block_table, Tensor query_start_loc, "
        "Tensor seq_lens, int pool, int max_query_len) -> ()");
  m.def("pooled_window_attention_rows(Tensor(a!) out, Tensor q, "
        "Tensor k_cache, Tensor v_cache, Tensor pool_k, Tensor pool_v, "
        "Tensor block_table, Tensor query_start_loc, Tensor seq_lens, "
        "Tensor? gate, float scale, int window, int pool, int row0, "
        "int num_rows) -> ()");
  m.def("pooled_window_attention_prefill(Tensor(a!) out, Tensor q, "
        "Tensor k_cache, Tensor v_cache, Tensor pool_k, Tensor pool_v, "
        "Tensor block_table, Tensor query_start_loc, Tensor seq_lens, "
        "Tensor? gate, float scale, int window, int pool, int num_decodes, "
        "int max_query_len) -> ()");
  m.def("pooled_window_attention_decode(Tensor(a!) out, Tensor q, "
        "Tensor k_cache, Tensor v_cache, Tensor pool_k, Tensor pool_v, "
        "Tensor block_table, Tensor query_start_loc, Tensor seq_lens, "
        "Tensor? gate, float scale, int window, int pool, int num_decodes, "
        "int max_seq_len) -> ()");
  m.def("scaled_embedding(Tensor ids, Tensor table, float scale) -> Tensor");
  m.def("rms_norm_cast(Tensor x, Tensor weight, float eps, "
        "ScalarType out_dtype) -> Tensor");
  m.def("add_rms_norm(Tensor(a!) residual, Tensor y, Tensor weight, "
        "float eps, ScalarType? out_dtype) -> Tensor");
  m.def("relu2(Tensor x) -> Tensor");
  m.def("logit_softcap(Tensor logits, float cap) -> Tensor");
  m.def("sigmoid_gate_mul(Tensor x, Tensor gate) -> Tensor");
  m.def("latent_rope_cache_write(Tensor(a!) q, Tensor? dkv, Tensor? norm_w, "
        "float eps, Tensor positions, Tensor inv_freq, int nope_dim, "
        "int kv_rank, Tensor(b!)? cache, Tensor? slot_mapping) -> ()");
  m.def("latent_attention_rows(Tensor(a!) out, Tensor q_abs, Tensor q_rot, "
        "Tensor cache, Tensor block_table, Tensor query_start_loc, "
        "Tensor seq_lens, Tensor? sink, float scale) -> ()");
  m.def("latent_attention_tiles_supported(int kv_rank, int rot_dim) -> bool");
  m.impl("latent_attention_tiles_supported",
         &vllm_amd::latent_attention_tiles_supported);
  m.def("latent_attention_tiles(Tensor(a!) out, Tensor q_abs, Tensor q_rot, "
        "Tensor cache, Tensor block_table, Tensor query_start_loc, "
        "Tensor seq_lens, Tensor? sink, float scale, int num_decodes, "
        "int max_seq_len) -> ()");
  m.def("causal_conv_silu(Tensor x, Tensor weight, Tensor bias, "
        "Tensor(a!)? conv_state, Tensor? state_rows, "
        "Tensor query_start_loc, ScalarType out_dtype) -> Tensor");
  m.def("ssd_scan(Tensor xbc, int heads, int head_dim, int groups, "
        "int state, Tensor dt, Tensor dt_bias, Tensor a_log, "
        "Tensor d_skip, Tensor(a!)? ssm_state, Tensor? state_rows, "
        "Tensor query_start_loc, int max_query_len) -> Tensor");
  m.def("gated_group_rms_norm(Tensor y, Tensor z, Tensor weight, "
        "float eps, int groups, ScalarType out_dtype) -> Tensor");
  // Custom xGMI collectives (comms.hip). init/connect/destroy are
  // host-side control ops and live on the catch-all dispatch below.
  m.def("car_init(int rank, int world, int max_bytes) -> Tensor");
  m.def("car_connect(Tensor handles) -> ()");
  m.def("car_is_ready() -> bool");
  m.def("car_max_bytes() -> int");
  m.def("car_error() -> int");
  m.def("car_destroy() -> ()");
  m.def("car_all_reduce(Tensor(a!) t) -> ()");
  m.def("car_all_gather(Tensor(a!) out, Tensor t) -> ()");
  m.def("car_reduce_scatter(Tensor(a!) out, Tensor t) -> ()");
  m.impl("car_init", &vllm_amd::car_init);
  m.impl("car_connect", &vllm_amd::car_connect);
  m.impl("car_is_ready", &vllm_amd::car_is_ready);
  m.impl("car_max_bytes", &vllm_amd::car_max_bytes);
  m.impl("car_error", &vllm_amd::car_error);
  m.impl("car_destroy", &vllm_amd::car_destroy);
}

TORCH_LIBRARY_IMPL(vllm_amd, CUDA, m) {
  m.impl("rms_norm", &vllm_amd::rms_norm);
  m.impl("fused_add_rms_norm", &vllm_amd::fused_add_rms_norm);
  m.impl("silu_and_mul", &vllm_amd::silu_and_mul);
  m.impl("gelu_and_mul", &vllm_amd::gelu_and_mul);
  m.impl("rotary_embedding", &vllm_amd::rotary_embedding);
  m.impl("reshape_and_cache", &vllm_amd::reshape_and_cache);
  m.impl("paged_decode_attention", &vllm_amd::paged_decode_attention);
  m.impl("prefill_attention", &vllm_amd::prefill_attention);
  m.impl("lt_linear", &vllm_amd::lt_linear);
  m.impl("lt_linear_fp8", &vllm_amd::lt_linear_fp8);
  m.impl("dynamic_quant_fp8", &vllm_amd::dynamic_quant_fp8);
  m.impl("scale_rows_cols", &vllm_amd::scale_rows_cols);
  m.impl("car_all_reduce", &vllm_amd::car_all_reduce);
  m.impl("car_all_gather", &vllm_amd::car_all_gather);
  m.impl("car_reduce_scatter", &vllm_amd::car_reduce_scatter);
  m.impl("moe_align", &vllm_amd::moe_align);
  m.impl("moe_gemm", &vllm_amd::moe_gemm);
  m.impl("moe_gemm_shuf", &vllm_amd::moe_gemm_shuf);
  m.impl("moe_combine", &vllm_amd::moe_combine);
  m.impl("mla_decode", &vllm_amd::mla_decode);
  m.impl("scalar_rms_norm", &vllm_amd::scalar_rms_norm);
  m.impl("add_scaled_scalar_norm", &vllm_amd::add_scaled_scalar_norm);
  m.impl("token_shift", &vllm_amd::token_shift);
  m.impl("silu_and_mul_any", &vllm_amd::silu_and_mul_any);
  m.impl("norm_qk_cache_write", &vllm_amd::norm_qk_cache_write);
  m.impl("pool_update", &vllm_amd::pool_update);
  m.impl("pooled_window_attention_prefill",
         &vllm_amd::pooled_window_attention_prefill);
  m.impl("pooled_window_attention_rows",
         &vllm_amd::pooled_window_attention_rows);
  m.impl("pooled_window_attention_decode",
         &vllm_amd::pooled_window_attention_decode);
  m.impl("scaled_embedding", &vllm_amd::scaled_embedding);
  m.impl("rms_norm_cast", &vllm_amd::rms_norm_cast);
  m.impl("add_rms_norm", &vllm_amd::add_rms_norm);
  m.impl("relu2", &vllm_amd::relu2);
  m.impl("logit_softcap", &vllm_amd::logit_softcap);
  m.impl("sigmoid_gate_mul", &vllm_amd::sigmoid_gate_mul);
  m.impl("latent_rope_cache_write", &vllm_amd::latent_rope_cache_write);
  m.impl("latent_attention_rows", &vllm_amd::latent_attention_rows);
  m.impl("latent_attention_tiles", &vllm_amd::latent_attention_tiles);
  m.impl("causal_conv_silu", &vllm_amd::causal_conv_silu);
  m.impl("ssd_scan", &vllm_amd::ssd_scan);
  m.impl("gated_group_rms_norm", &vllm_amd::gated_group_rms_norm);
}
