// Python bindings for the hybrid-decoder kernel library (gfx950): the
// mechanisms behind recurrent / latent-attention layers.  Built as its own
// extension so a process that serves such a model compiles and loads only
// these kernels.
#include <torch/extension.h>

namespace igw {
void add_layernorm(torch::Tensor out, torch::Tensor residual,
                   c10::optional<torch::Tensor> delta, torch::Tensor weight,
                   torch::Tensor bias, double eps);
void latent_down_post(torch::Tensor cq, torch::Tensor gate, torch::Tensor down,
                      torch::Tensor positions, torch::Tensor slot_mapping,
                      torch::Tensor cache, torch::Tensor qnorm_w,
                      torch::Tensor kvnorm_w, torch::Tensor inv_freq,
                      double eps, int64_t q_rank, int64_t kv_rank,
                      int64_t rot_dim, int64_t heads);
void rope_pairs(torch::Tensor x, torch::Tensor positions,
                torch::Tensor inv_freq, int64_t offset);
void xielu(torch::Tensor out, torch::Tensor in, torch::Tensor pq);
void relu2(torch::Tensor out, torch::Tensor in);
void gate_heads(torch::Tensor out, torch::Tensor v, torch::Tensor gate);
void moe_topk_route(torch::Tensor weights, torch::Tensor idx,
                    torch::Tensor logits, c10::optional<torch::Tensor> dst,
                    c10::optional<torch::Tensor> counts, int64_t capacity,
                    double scale);
void add_rmsnorm_pair(torch::Tensor out1, c10::optional<torch::Tensor> out2,
                      torch::Tensor residual,
                      c10::optional<torch::Tensor> delta_a,
                      c10::optional<torch::Tensor> delta_b, torch::Tensor w1,
                      c10::optional<torch::Tensor> w2, double eps);
void qk_norm_append(torch::Tensor q_out, torch::Tensor proj,
                    torch::Tensor slot_mapping, torch::Tensor kcache,
                    torch::Tensor vcache, torch::Tensor qnorm_w,
                    torch::Tensor knorm_w,
                    c10::optional<torch::Tensor> v_first, double lam,
                    double eps, int64_t heads, int64_t kv_heads, int64_t dim,
                    int64_t vdim);
void gated_act(torch::Tensor out, torch::Tensor in, int64_t mode, double limit,
               double alpha);
void sigmoid_attention(torch::Tensor out, torch::Tensor q,
                       torch::Tensor kcache, torch::Tensor vcache,
                       torch::Tensor block_table, torch::Tensor row_seq,
                       torch::Tensor positions, torch::Tensor dist_bias,
                       torch::Tensor talk, torch::Tensor gate, double scale,
                       int64_t window);
void mingru_scan(torch::Tensor y, torch::Tensor zug, torch::Tensor state,
                 torch::Tensor seq_cu, torch::Tensor seq_start,
                 torch::Tensor seq_slots);
void mingru_scan_chunked(torch::Tensor y, torch::Tensor zug,
                         torch::Tensor state, torch::Tensor seq_start,
                         torch::Tensor seq_slots, torch::Tensor chunk_r0,
                         torch::Tensor chunk_r1, torch::Tensor seq_chunk_cu,
                         torch::Tensor work);
void latent_attention(torch::Tensor out, torch::Tensor q_abs,
                      torch::Tensor q_rot, torch::Tensor cache,
                      torch::Tensor block_table, torch::Tensor row_seq,
                      torch::Tensor positions, torch::Tensor sink,
                      double scale, int64_t window);
bool latent_attention_mfma(torch::Tensor out, torch::Tensor q_abs,
                           torch::Tensor q_rot, torch::Tensor cache,
                           torch::Tensor block_table, torch::Tensor row_seq,
                           torch::Tensor positions, torch::Tensor tile_row0,
                           torch::Tensor tile_nrows, torch::Tensor sink,
                           double scale, int64_t window, int64_t max_keys);
int64_t latent_attention_tile_rows(int64_t H);
bool sigmoid_attention_mfma(torch::Tensor out, torch::Tensor q,
                            torch::Tensor kcache, torch::Tensor vcache,
                            torch::Tensor block_table, torch::Tensor row_seq,
                            torch::Tensor positions, torch::Tensor tile_row0,
                            torch::Tensor tile_nrows, torch::Tensor dist_bias,
                            torch::Tensor talk, torch::Tensor gate,
                            double scale, int64_t window, int64_t max_keys,
                            int64_t num_prefill_rows);
int64_t sigmoid_attention_tile_rows();
}  // namespace igw

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.def("add_layernorm", &igw::add_layernorm,
        "fp32 residual += delta; LayerNorm with weight and bias");
  m.def("latent_down_post", &igw::latent_down_post,
        "latent RMS norms + shared-key rotation + paged append + head gates");
  m.def("rope_pairs", &igw::rope_pairs,
        "in-place interleaved-pair rotary on a slice of every head");
  m.def("xielu", &igw::xielu, "xIELU activation");
  m.def("relu2", &igw::relu2, "squared ReLU activation");
  m.def("gate_heads", &igw::gate_heads,
        "[H,T,vd] values times [T,H] gates -> [T,H*vd]");
  m.def("moe_topk_route", &igw::moe_topk_route,
        "top-k experts and softmax over the chosen logits");
  m.def("add_rmsnorm_pair", &igw::add_rmsnorm_pair,
        "fp32 residual += two deltas; one RMS statistic, two weighted outputs");
  m.def("qk_norm_append", &igw::qk_norm_append,
        "whole-projection query/key RMS norms + value blend + paged append");
  m.def("gated_act", &igw::gated_act,
        "(gate | up) -> silu(g) u or the clamped gated unit");
  m.def("sigmoid_attention", &igw::sigmoid_attention,
        "windowed sigmoid attention, distance bias, head mixing, paged");
  m.def("sigmoid_attention_mfma", &igw::sigmoid_attention_mfma,
        "windowed sigmoid attention on MFMA tiles (bf16); false = sizes do "
        "not fit, use sigmoid_attention");
  m.def("sigmoid_attention_tile_rows", &igw::sigmoid_attention_tile_rows,
        "token rows per MFMA tile");
  m.def("mingru_scan", &igw::mingru_scan,
        "minGRU recurrence, one thread per (sequence, channel)");
  m.def("mingru_scan_chunked", &igw::mingru_scan_chunked,
        "minGRU recurrence as a three-pass chunked scan");
  m.def("latent_attention", &igw::latent_attention,
        "absorbed latent attention, sliding window + softmax sink, paged");
  m.def("latent_attention_mfma", &igw::latent_attention_mfma,
        "absorbed latent attention on MFMA tiles (bf16); false = sizes do "
        "not fit, use latent_attention");
  m.def("latent_attention_tile_rows", &igw::latent_attention_tile_rows,
        "token rows per MFMA tile for a head count");
}
