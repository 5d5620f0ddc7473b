// Python bindings of the ragged-batch sequence kernels.
#include <torch/extension.h>

torch::Tensor embed_tokens(torch::Tensor tokens, torch::Tensor cu, torch::Tensor slots, torch::Tensor tok_req,
                           torch::Tensor tok_pos, torch::Tensor embed, torch::Tensor bigram, torch::Tensor pos,
                           torch::Tensor prev_state, int64_t mul_prev, int64_t mul_cur, int64_t buckets);
torch::Tensor hc_mix_norm(torch::Tensor streams, torch::Tensor y, torch::Tensor mix, torch::Tensor out_w,
                          torch::Tensor in_w, torch::Tensor norm_w, double eps);
torch::Tensor canon_conv(torch::Tensor h, torch::Tensor w, torch::Tensor state, torch::Tensor cu,
                         torch::Tensor slots, torch::Tensor tok_req, bool out_bf16);
torch::Tensor xielu(torch::Tensor z, torch::Tensor act);
torch::Tensor gate_heads(torch::Tensor x, torch::Tensor g, int64_t H);
torch::Tensor rmsnorm_rows(torch::Tensor x, torch::Tensor w, double eps);
torch::Tensor mingru_scan(torch::Tensor zxg, torch::Tensor bz, torch::Tensor bx, torch::Tensor state,
                          torch::Tensor cu, torch::Tensor slots);
torch::Tensor mlstm_scan(torch::Tensor qkvg, torch::Tensor gates, torch::Tensor bi, torch::Tensor bfg,
                         torch::Tensor norm_w, int64_t H, int64_t D, int64_t V, double cap, double eps,
                         torch::Tensor stS, torch::Tensor stn, torch::Tensor stm, torch::Tensor cu,
                         torch::Tensor slots);
void latent_kv_store(torch::Tensor dkv, torch::Tensor w, double eps, torch::Tensor cosv, torch::Tensor sinv,
                     int64_t rot_dims, int64_t rank, torch::Tensor pool, torch::Tensor tok_pos,
                     torch::Tensor tok_row);
torch::Tensor assemble_latent_q(torch::Tensor qa, torch::Tensor qr, torch::Tensor cosv, torch::Tensor sinv,
                                int64_t rot_dims, torch::Tensor tok_pos);
torch::Tensor latent_sink_attention(torch::Tensor q, torch::Tensor pool, int64_t rank, torch::Tensor sink,
                                    double scale, torch::Tensor tok_req, torch::Tensor tok_pos,
                                    torch::Tensor tables, int64_t bs);
torch::Tensor latent_sink_attention_mfma(torch::Tensor q, torch::Tensor pool, int64_t rank, torch::Tensor sink,
                                         double scale, torch::Tensor tiles, torch::Tensor cu, torch::Tensor start_pos,
                                         torch::Tensor tables, int64_t bs, int64_t nsplit);

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.def("embed_tokens", &embed_tokens);
  m.def("hc_mix_norm", &hc_mix_norm);
  m.def("canon_conv", &canon_conv);
  m.def("xielu", &xielu);
  m.def("gate_heads", &gate_heads);
  m.def("rmsnorm_rows", &rmsnorm_rows);
  m.def("mingru_scan", &mingru_scan);
  m.def("mlstm_scan", &mlstm_scan);
  m.def("latent_kv_store", &latent_kv_store);
  m.def("assemble_latent_q", &assemble_latent_q);
  m.def("latent_sink_attention", &latent_sink_attention);
  m.def("latent_sink_attention_mfma", &latent_sink_attention_mfma);
}
