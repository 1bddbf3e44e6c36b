// Operator schemas and registrations of torch.ops.llmctl_hybrid.* (kernels: the .hip files beside
// this one; CUDA dispatch key == HIP on ROCm builds of PyTorch).
#include <torch/library.h>
#include <ATen/ATen.h>

namespace llmctl_hybrid {
at::Tensor layernorm_f32(const at::Tensor& x, const at::Tensor& w, const at::Tensor& b, double eps, bool out_bf16);
void residual_add_(at::Tensor x, const at::Tensor& a, const c10::optional<at::Tensor>& b);
at::Tensor add_layernorm_f32_(at::Tensor x, const at::Tensor& a, const c10::optional<at::Tensor>& b, const at::Tensor& w,
                              const at::Tensor& bias, double eps, bool out_bf16);
at::Tensor rmsnorm_cols(const at::Tensor& x, const at::Tensor& w, double eps, int64_t n, bool out_bf16);
at::Tensor sigmoid_gate_mul(const at::Tensor& o, const at::Tensor& g);
at::Tensor swiglu_any(const at::Tensor& gu);
at::Tensor headnorm_gate(const at::Tensor& o, const at::Tensor& w, const at::Tensor& g, double eps, bool out_bf16, bool silu);
void latent_kv_write(const at::Tensor& dkv, const at::Tensor& norm_w, double eps, const at::Tensor& pos, const at::Tensor& inv_freq,
                     int64_t rot_dims, at::Tensor cache, const at::Tensor& slots, bool interleaved, double amp);
at::Tensor latent_q_assemble(const at::Tensor& q_lat, const at::Tensor& q, const at::Tensor& pos, const at::Tensor& inv_freq,
                             int64_t rot_dims, int64_t dn, bool interleaved, double amp);
at::Tensor latent_attn_prefill(const at::Tensor& qa, const at::Tensor& cache, const at::Tensor& bt, const at::Tensor& cu,
                               const at::Tensor& ctx, int64_t window, const c10::optional<at::Tensor>& sink, double scale, int64_t rk,
                               int64_t max_q, bool mfma, int64_t groups, int64_t koff, int64_t chunk,
                               const c10::optional<at::Tensor>& hscale, const c10::optional<at::Tensor>& ofreq,
                               const c10::optional<at::Tensor>& sig_bias, const c10::optional<at::Tensor>& dist_a,
                               const c10::optional<at::Tensor>& dist_b, double softcap, int64_t keep_first);
at::Tensor latent_attn_decode(const at::Tensor& qa, const at::Tensor& cache, const at::Tensor& bt, const at::Tensor& ctx,
                              int64_t window, const c10::optional<at::Tensor>& sink, double scale, int64_t rk, bool mfma, int64_t groups,
                              int64_t koff, int64_t chunk, const c10::optional<at::Tensor>& hscale, const c10::optional<at::Tensor>& ofreq,
                              int64_t max_ctx, const c10::optional<at::Tensor>& sig_bias, const c10::optional<at::Tensor>& dist_a,
                              const c10::optional<at::Tensor>& dist_b, double softcap, int64_t keep_first);
std::tuple<at::Tensor, at::Tensor> add_rmsnorm2_f32_(at::Tensor x, const c10::optional<at::Tensor>& a, const c10::optional<at::Tensor>& b,
                                                     const at::Tensor& w1, const c10::optional<at::Tensor>& w2, double eps, bool one_plus,
                                                     bool out_bf16);
void residual_add_act_(at::Tensor x, const at::Tensor& a, const c10::optional<at::Tensor>& b);
at::Tensor clamped_glu(const at::Tensor& gu, double limit, double alpha);
at::Tensor causal_conv(const at::Tensor& u, const at::Tensor& w, at::Tensor state, const at::Tensor& seq_of, const at::Tensor& cu,
                       const at::Tensor& start, const at::Tensor& sslot, bool add_input, int64_t max_len);
at::Tensor attn_qkv_prep(const at::Tensor& z, int64_t H, int64_t G, int64_t dk, int64_t dv, const c10::optional<at::Tensor>& q_norm,
                         const c10::optional<at::Tensor>& k_norm, double eps, const at::Tensor& pos, const at::Tensor& freq, int64_t rot_dims,
                         bool interleaved, double amp, const c10::optional<at::Tensor>& vfreq, at::Tensor cache, const at::Tensor& slots,
                         bool v_from_k, const c10::optional<at::Tensor>& v_first, const c10::optional<at::Tensor>& v_lambda);
at::Tensor mlstm_scan(const at::Tensor& q, const at::Tensor& k, const at::Tensor& v, const at::Tensor& gates, const at::Tensor& b_i,
                      const at::Tensor& b_f, double cap, double qscale, at::Tensor S, at::Tensor n, at::Tensor m,
                      const at::Tensor& slots, const at::Tensor& cu, const at::Tensor& start, bool slab,
                      const c10::optional<at::Tensor>& fsum, bool write_out);
void mlstm_chunk_combine(const at::Tensor& S, const at::Tensor& n, const at::Tensor& m, const at::Tensor& slots, const at::Tensor& start,
                         const at::Tensor& base, const at::Tensor& locS, const at::Tensor& locn, const at::Tensor& locm,
                         const at::Tensor& fsum, at::Tensor iS, at::Tensor in_, at::Tensor im);
std::tuple<at::Tensor, at::Tensor> group_topk_router(const at::Tensor& logits, int64_t top, int64_t groups, int64_t keep);
std::tuple<at::Tensor, at::Tensor> bias_topk_router(const at::Tensor& logits, const c10::optional<at::Tensor>& bias, int64_t top, int64_t groups,
                                                    int64_t keep, bool renorm);
std::tuple<at::Tensor, at::Tensor> hc_embed_norm(const at::Tensor& ids, const at::Tensor& table, int64_t streams, const at::Tensor& c_in,
                                                 const at::Tensor& g, double eps, bool out_bf16);
at::Tensor hc_update_norm_(at::Tensor X, const at::Tensor& y1, double s1, const c10::optional<at::Tensor>& y2, double s2, const at::Tensor& mix,
                           const at::Tensor& c_out, double mult, const c10::optional<at::Tensor>& c_in, const c10::optional<at::Tensor>& g,
                           double eps, bool out_bf16);
void gated_add_f32_(at::Tensor out, const at::Tensor& y, const at::Tensor& g);
at::Tensor tanh_act(const at::Tensor& x);
void softcap_(at::Tensor x, double cap);
at::Tensor delta_scan(const at::Tensor& r, const at::Tensor& k, const at::Tensor& v, const at::Tensor& zw, const at::Tensor& w0,
                      const at::Tensor& za, const at::Tensor& ab, double decay_coef, double key_eps, at::Tensor S, const at::Tensor& slots,
                      const at::Tensor& cu, const at::Tensor& start, const c10::optional<at::Tensor>& P, bool write_out, bool write_state);
void delta_chunk_combine(at::Tensor S, const at::Tensor& slots, const at::Tensor& start, const at::Tensor& base, const at::Tensor& loc,
                         const at::Tensor& P, at::Tensor init);
at::Tensor gated_norm_add_norm_f32_(at::Tensor x, const at::Tensor& y, const at::Tensor& r, const at::Tensor& w_post,
                                    const c10::optional<at::Tensor>& w_next, double eps, bool out_bf16);
std::tuple<at::Tensor, at::Tensor> embed_rmsnorm_f32(const at::Tensor& ids, const at::Tensor& pos, const at::Tensor& table,
                                                     const at::Tensor& pos_table, const at::Tensor& w, double eps, bool out_bf16);
at::Tensor act_any(const at::Tensor& x, int64_t kind);
at::Tensor qk_fullnorm_prep(const at::Tensor& z, int64_t H, int64_t G, int64_t dk, int64_t dv, const at::Tensor& q_norm, const at::Tensor& k_norm,
                            double eps, const at::Tensor& pos, double temp_coef, int64_t temp_every, at::Tensor cache, const at::Tensor& slots);
at::Tensor gla_scan(const at::Tensor& q, const at::Tensor& k, const at::Tensor& v, const at::Tensor& z, const at::Tensor& z_bias,
                    double tau, double qscale, at::Tensor S, const at::Tensor& slots, const at::Tensor& cu, const at::Tensor& start,
                    const c10::optional<at::Tensor>& logd, bool write_out, bool write_state);
void gla_chunk_combine(at::Tensor S, const at::Tensor& slots, const at::Tensor& start, const at::Tensor& base, const at::Tensor& loc,
                       const at::Tensor& logd, at::Tensor init);
}  // namespace llmctl_hybrid

TORCH_LIBRARY(llmctl_hybrid, m) {
  m.def("layernorm_f32(Tensor x, Tensor w, Tensor b, float eps, bool out_bf16) -> Tensor");
  m.def("residual_add_(Tensor(a!) x, Tensor a, Tensor? b) -> ()");
  m.def("add_layernorm_f32_(Tensor(a!) x, Tensor a, Tensor? b, Tensor w, Tensor bias, float eps, bool out_bf16) -> Tensor");
  m.def("rmsnorm_cols(Tensor x, Tensor w, float eps, int n, bool out_bf16) -> Tensor");
  m.def("sigmoid_gate_mul(Tensor o, Tensor g) -> Tensor");
  m.def("swiglu_any(Tensor gu) -> Tensor");
  m.def("headnorm_gate(Tensor o, Tensor w, Tensor g, float eps, bool out_bf16, bool silu=False) -> Tensor");
  m.def("latent_kv_write(Tensor dkv, Tensor norm_w, float eps, Tensor pos, Tensor inv_freq, int rot_dims, Tensor(a!) cache, Tensor slots, bool interleaved=False, float amp=1.0) -> ()");
  m.def("latent_q_assemble(Tensor q_lat, Tensor q, Tensor pos, Tensor inv_freq, int rot_dims, int dn, bool interleaved=False, float amp=1.0) -> Tensor");
  m.def("latent_attn_prefill(Tensor qa, Tensor cache, Tensor bt, Tensor cu, Tensor ctx, int window, Tensor? sink, float scale, int rk, int max_q, bool mfma=True, int groups=1, int koff=0, int chunk=1073741824, Tensor? hscale=None, Tensor? ofreq=None, Tensor? sig_bias=None, Tensor? dist_a=None, Tensor? dist_b=None, float softcap=0.0, int keep_first=0) -> Tensor");
  m.def("latent_attn_decode(Tensor qa, Tensor cache, Tensor bt, Tensor ctx, int window, Tensor? sink, float scale, int rk, bool mfma=True, int groups=1, int koff=0, int chunk=1073741824, Tensor? hscale=None, Tensor? ofreq=None, int max_ctx=0, Tensor? sig_bias=None, Tensor? dist_a=None, Tensor? dist_b=None, float softcap=0.0, int keep_first=0) -> Tensor");
  m.def("add_rmsnorm2_f32_(Tensor(a!) x, Tensor? a, Tensor? b, Tensor w1, Tensor? w2, float eps, bool one_plus, bool out_bf16) -> (Tensor, Tensor)");
  m.def("residual_add_act_(Tensor(a!) x, Tensor a, Tensor? b) -> ()");
  m.def("clamped_glu(Tensor gu, float limit, float alpha) -> Tensor");
  m.def("causal_conv(Tensor u, Tensor w, Tensor(a!) state, Tensor seq_of, Tensor cu, Tensor start, Tensor sslot, bool add_input, int max_len=0) -> Tensor");
  m.def("attn_qkv_prep(Tensor z, int H, int G, int dk, int dv, Tensor? q_norm, Tensor? k_norm, float eps, Tensor pos, Tensor freq, int rot_dims, bool interleaved, float amp, Tensor? vfreq, Tensor(a!) cache, Tensor slots, bool v_from_k=False, Tensor? v_first=None, Tensor? v_lambda=None) -> Tensor");
  m.def("mlstm_scan(Tensor q, Tensor k, Tensor v, Tensor gates, Tensor b_i, Tensor b_f, float cap, float qscale, Tensor(a!) S, Tensor(b!) n, Tensor(c!) m, Tensor slots, Tensor cu, Tensor start, bool slab=False, Tensor(d!)? fsum=None, bool write_out=True) -> Tensor");
  m.def("mlstm_chunk_combine(Tensor S, Tensor n, Tensor m, Tensor slots, Tensor start, Tensor base, Tensor locS, Tensor locn, Tensor locm, Tensor fsum, Tensor(a!) iS, Tensor(b!) in_, Tensor(c!) im) -> ()");
  m.def("group_topk_router(Tensor logits, int top, int groups, int keep) -> (Tensor, Tensor)");
  m.def("bias_topk_router(Tensor logits, Tensor? bias, int top, int groups=1, int keep=1, bool renorm=True) -> (Tensor, Tensor)");
  m.def("hc_embed_norm(Tensor ids, Tensor table, int streams, Tensor c_in, Tensor g, float eps, bool out_bf16) -> (Tensor, Tensor)");
  m.def("hc_update_norm_(Tensor(a!) X, Tensor y1, float s1, Tensor? y2, float s2, Tensor mix, Tensor c_out, float mult, Tensor? c_in, Tensor? g, float eps, bool out_bf16) -> Tensor");
  m.def("gated_add_f32_(Tensor(a!) out, Tensor y, Tensor g) -> ()");
  m.def("tanh_act(Tensor x) -> Tensor");
  m.def("softcap_(Tensor(a!) x, float cap) -> ()");
  m.def("delta_scan(Tensor r, Tensor k, Tensor v, Tensor zw, Tensor w0, Tensor za, Tensor ab, float decay_coef, float key_eps, Tensor(a!) S, Tensor slots, Tensor cu, Tensor start, Tensor(b!)? P=None, bool write_out=True, bool write_state=True) -> Tensor");
  m.def("delta_chunk_combine(Tensor(a!) S, Tensor slots, Tensor start, Tensor base, Tensor loc, Tensor P, Tensor(b!) init) -> ()");
  m.def("gated_norm_add_norm_f32_(Tensor(a!) x, Tensor y, Tensor r, Tensor w_post, Tensor? w_next, float eps, bool out_bf16) -> Tensor");
  m.def("embed_rmsnorm_f32(Tensor ids, Tensor pos, Tensor table, Tensor pos_table, Tensor w, float eps, bool out_bf16) -> (Tensor, Tensor)");
  m.def("act_any(Tensor x, int kind) -> Tensor");
  m.def("qk_fullnorm_prep(Tensor z, int H, int G, int dk, int dv, Tensor q_norm, Tensor k_norm, float eps, Tensor pos, float temp_coef, int temp_every, Tensor(a!) cache, Tensor slots) -> Tensor");
  m.def("gla_scan(Tensor q, Tensor k, Tensor v, Tensor z, Tensor z_bias, float tau, float qscale, Tensor(a!) S, Tensor slots, Tensor cu, Tensor start, Tensor(b!)? logd=None, bool write_out=True, bool write_state=True) -> Tensor");
  m.def("gla_chunk_combine(Tensor(a!) S, Tensor slots, Tensor start, Tensor base, Tensor loc, Tensor logd, Tensor(b!) init) -> ()");
}

TORCH_LIBRARY_IMPL(llmctl_hybrid, CUDA, m) {
  m.impl("layernorm_f32", &llmctl_hybrid::layernorm_f32);
  m.impl("residual_add_", &llmctl_hybrid::residual_add_);
  m.impl("add_layernorm_f32_", &llmctl_hybrid::add_layernorm_f32_);
  m.impl("rmsnorm_cols", &llmctl_hybrid::rmsnorm_cols);
  m.impl("sigmoid_gate_mul", &llmctl_hybrid::sigmoid_gate_mul);
  m.impl("swiglu_any", &llmctl_hybrid::swiglu_any);
  m.impl("headnorm_gate", &llmctl_hybrid::headnorm_gate);
  m.impl("latent_kv_write", &llmctl_hybrid::latent_kv_write);
  m.impl("latent_q_assemble", &llmctl_hybrid::latent_q_assemble);
  m.impl("latent_attn_prefill", &llmctl_hybrid::latent_attn_prefill);
  m.impl("latent_attn_decode", &llmctl_hybrid::latent_attn_decode);
  m.impl("add_rmsnorm2_f32_", &llmctl_hybrid::add_rmsnorm2_f32_);
  m.impl("residual_add_act_", &llmctl_hybrid::residual_add_act_);
  m.impl("clamped_glu", &llmctl_hybrid::clamped_glu);
  m.impl("causal_conv", &llmctl_hybrid::causal_conv);
  m.impl("attn_qkv_prep", &llmctl_hybrid::attn_qkv_prep);
  m.impl("mlstm_scan", &llmctl_hybrid::mlstm_scan);
  m.impl("mlstm_chunk_combine", &llmctl_hybrid::mlstm_chunk_combine);
  m.impl("group_topk_router", &llmctl_hybrid::group_topk_router);
  m.impl("bias_topk_router", &llmctl_hybrid::bias_topk_router);
  m.impl("gated_norm_add_norm_f32_", &llmctl_hybrid::gated_norm_add_norm_f32_);
  m.impl("embed_rmsnorm_f32", &llmctl_hybrid::embed_rmsnorm_f32);
  m.impl("act_any", &llmctl_hybrid::act_any);
  m.impl("qk_fullnorm_prep", &llmctl_hybrid::qk_fullnorm_prep);
  m.impl("gla_scan", &llmctl_hybrid::gla_scan);
  m.impl("gla_chunk_combine", &llmctl_hybrid::gla_chunk_combine);
  m.impl("hc_embed_norm", &llmctl_hybrid::hc_embed_norm);
  m.impl("hc_update_norm_", &llmctl_hybrid::hc_update_norm_);
  m.impl("gated_add_f32_", &llmctl_hybrid::gated_add_f32_);
  m.impl("tanh_act", &llmctl_hybrid::tanh_act);
  m.impl("softcap_", &llmctl_hybrid::softcap_);
  m.impl("delta_scan", &llmctl_hybrid::delta_scan);
  m.impl("delta_chunk_combine", &llmctl_hybrid::delta_chunk_combine);
}
