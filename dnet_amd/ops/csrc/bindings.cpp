// Python bindings for the dnet_amd gfx950 kernel extension.
#include <torch/extension.h>
namespace py = pybind11;

namespace dnet {
void rmsnorm_f32(torch::Tensor xf, torch::Tensor residual, torch::Tensor w,
                 torch::Tensor y, double eps);
void resid_add_f32(torch::Tensor h, torch::Tensor xf);
void rmsnorm(torch::Tensor x, c10::optional<torch::Tensor> residual,
             torch::Tensor w, torch::Tensor y, double eps);
void gemv_bf16(torch::Tensor x, torch::Tensor w, torch::Tensor out,
               c10::optional<torch::Tensor> bias);
void gemv_int8(torch::Tensor x, torch::Tensor w, torch::Tensor scales,
               torch::Tensor out, int64_t group,
               c10::optional<torch::Tensor> bias, bool packed);
void attn_decode(torch::Tensor q, torch::Tensor kcache, torch::Tensor vcache,
                 torch::Tensor pos, torch::Tensor out, double scale,
                 int64_t window, c10::optional<torch::Tensor> sinks,
                 c10::optional<torch::Tensor> kscale,
                 c10::optional<torch::Tensor> vscale,
                 c10::optional<torch::Tensor> partials, int64_t splits,
                 bool combine);
void attn_prefill(torch::Tensor q, torch::Tensor k, torch::Tensor v,
                  c10::optional<torch::Tensor> sinks, torch::Tensor out,
                  int64_t q_off, int64_t window, double scale);
void attn_combine(torch::Tensor partials, c10::optional<torch::Tensor> sinks,
                  torch::Tensor out, int64_t splits);
void rope_append_f32(torch::Tensor src, c10::optional<torch::Tensor> bias,
                     torch::Tensor qout, int64_t Hkv, torch::Tensor kcache,
                     torch::Tensor vcache, torch::Tensor pos,
                     torch::Tensor cos_table, torch::Tensor sin_table,
                     c10::optional<torch::Tensor> kscale,
                     c10::optional<torch::Tensor> vscale,
                     c10::optional<torch::Tensor> wpos);
void rope_append(torch::Tensor q, torch::Tensor k, torch::Tensor v,
                 torch::Tensor kcache, torch::Tensor vcache, torch::Tensor pos,
                 torch::Tensor cos_table, torch::Tensor sin_table,
                 c10::optional<torch::Tensor> kscale,
                 c10::optional<torch::Tensor> vscale,
                 c10::optional<torch::Tensor> wpos);
void swiglu(torch::Tensor gu, torch::Tensor y);
void swiglu_f32(torch::Tensor gu_f32, torch::Tensor y, int64_t N);
void dequant_int8(torch::Tensor w, torch::Tensor scales, torch::Tensor out,
                  int64_t group, bool packed);
void dequant_int4(torch::Tensor w, torch::Tensor scales, torch::Tensor out,
                  int64_t group);
void dequant_mxfp4(torch::Tensor w, torch::Tensor scales, torch::Tensor out);
void scratch_clean(torch::Tensor scratch);
bool gemm_m16_will_defer(int64_t M, int64_t N, int64_t K, int64_t group,
                         int64_t bits, int64_t scratch_elems);
bool gemm_m16(torch::Tensor x, torch::Tensor w,
              c10::optional<torch::Tensor> scales,
              c10::optional<torch::Tensor> bias, torch::Tensor out,
              c10::optional<torch::Tensor> scratch, int64_t group, bool packed,
              int64_t bits, bool defer_combine);
void moe_gateup(torch::Tensor x, torch::Tensor w,
                c10::optional<torch::Tensor> scales,
                c10::optional<torch::Tensor> bias, torch::Tensor we,
                torch::Tensor act, int64_t group, bool packed, int64_t glu,
                double alpha, double limit);
void moe_down(torch::Tensor act, torch::Tensor w,
              c10::optional<torch::Tensor> scales,
              c10::optional<torch::Tensor> bias, torch::Tensor we,
              torch::Tensor out, int64_t group, bool packed);
void col_norm2(torch::Tensor x, torch::Tensor norms);
void gather_cols(torch::Tensor x, torch::Tensor idx, torch::Tensor out);
void scatter_cols(torch::Tensor in, torch::Tensor idx, torch::Tensor out);
void rmsnorm_rows(torch::Tensor x, torch::Tensor w, torch::Tensor y,
                  double eps);
void ls_resid_rmsnorm(torch::Tensor h, torch::Tensor a, torch::Tensor s1,
                      c10::optional<torch::Tensor> b,
                      c10::optional<torch::Tensor> s2,
                      c10::optional<torch::Tensor> wn,
                      c10::optional<torch::Tensor> y, double eps);
void xielu(torch::Tensor z, torch::Tensor pq, torch::Tensor y);
void qknorm_append(torch::Tensor qkv, torch::Tensor qw, torch::Tensor kw,
                   torch::Tensor qout, torch::Tensor kcache,
                   torch::Tensor vcache, torch::Tensor pos,
                   c10::optional<torch::Tensor> lens,
                   c10::optional<torch::Tensor> slots, double eps, int64_t nq,
                   int64_t nkv, int64_t d, int64_t dv, int64_t T,
                   bool per_head, c10::optional<torch::Tensor> rot_freq);
void resid_branches_rmsnorm(torch::Tensor h, torch::Tensor a,
                            c10::optional<torch::Tensor> wa,
                            c10::optional<torch::Tensor> b,
                            c10::optional<torch::Tensor> wb, double coef,
                            c10::optional<torch::Tensor> f,
                            c10::optional<torch::Tensor> wn,
                            c10::optional<torch::Tensor> y,
                            c10::optional<torch::Tensor> xc, double eps);
void gated_group_rmsnorm(torch::Tensor y, torch::Tensor gate_src,
                         int64_t gate_col0, torch::Tensor w, torch::Tensor out,
                         int64_t groups, double eps, bool gate_silu,
                         bool gate_first);
void act_slice(torch::Tensor x, int64_t col0, torch::Tensor y, int64_t kind);
void gelu_gather_mul(torch::Tensor z, torch::Tensor table,
                     torch::Tensor tokens, int64_t col0, torch::Tensor y);
void clamped_glu(torch::Tensor gu, torch::Tensor y, double alpha,
                 double limit);
void kv_pool_update(torch::Tensor kcache, torch::Tensor vcache,
                    torch::Tensor pool_k, torch::Tensor pool_v,
                    torch::Tensor pos, c10::optional<torch::Tensor> lens,
                    c10::optional<torch::Tensor> slots, int64_t T,
                    int64_t pool);
void causal_conv_silu(torch::Tensor x, int64_t col0, torch::Tensor w,
                      torch::Tensor bias, torch::Tensor state, torch::Tensor y,
                      torch::Tensor pos, c10::optional<torch::Tensor> lens,
                      c10::optional<torch::Tensor> slots, int64_t T);
void ssd_scan(torch::Tensor xbc, torch::Tensor dt_src, int64_t dt_col0,
              torch::Tensor dt_bias, torch::Tensor a_log, torch::Tensor dskip,
              torch::Tensor state, torch::Tensor y, torch::Tensor pos,
              c10::optional<torch::Tensor> lens,
              c10::optional<torch::Tensor> slots, int64_t T, int64_t heads,
              int64_t P, int64_t N, int64_t G);
void delta_scan(torch::Tensor src, int64_t r0, int64_t k0, int64_t v0,
                int64_t a0, torch::Tensor wl, torch::Tensor w0,
                torch::Tensor ab, torch::Tensor state, torch::Tensor o,
                torch::Tensor pos, c10::optional<torch::Tensor> lens,
                c10::optional<torch::Tensor> slots, int64_t T, int64_t H,
                int64_t d, double decay_scale, double unit_eps);
void attn_mod(torch::Tensor q, torch::Tensor kcache,
              c10::optional<torch::Tensor> vcache,
              torch::Tensor pos, c10::optional<torch::Tensor> lens,
              c10::optional<torch::Tensor> slots, torch::Tensor out,
              int64_t T, double scale, c10::optional<torch::Tensor> temp,
              double softcap, c10::optional<torch::Tensor> dist_r1,
              c10::optional<torch::Tensor> dist_r2,
              c10::optional<torch::Tensor> sinks, int64_t window,
              c10::optional<torch::Tensor> partials, int64_t splits,
              c10::optional<torch::Tensor> pool_k,
              c10::optional<torch::Tensor> pool_v, int64_t pool,
              int64_t v_dim, int64_t chunk,
              c10::optional<torch::Tensor> sig_bias);
void pair_hash_embed(torch::Tensor tokens, torch::Tensor embed,
                     torch::Tensor table, torch::Tensor prev,
                     torch::Tensor out, torch::Tensor pos,
                     c10::optional<torch::Tensor> lens,
                     c10::optional<torch::Tensor> slots, int64_t buckets,
                     int64_t mul_prev, int64_t mul_cur);
void causal_conv_residual(torch::Tensor x, torch::Tensor w, torch::Tensor state,
                          torch::Tensor y, torch::Tensor pos,
                          c10::optional<torch::Tensor> lens,
                          c10::optional<torch::Tensor> slots, int64_t T);
void decay_scan(torch::Tensor src, int64_t q0, int64_t k0, int64_t v0,
                torch::Tensor decay, torch::Tensor state, torch::Tensor o,
                torch::Tensor pos, c10::optional<torch::Tensor> lens,
                c10::optional<torch::Tensor> slots, int64_t T, int64_t H,
                int64_t d, int64_t dv);
void qknorm_half_append(torch::Tensor qk, torch::Tensor qw, torch::Tensor kw,
                        torch::Tensor qout, torch::Tensor kcache,
                        torch::Tensor vcache, torch::Tensor pos,
                        c10::optional<torch::Tensor> lens,
                        c10::optional<torch::Tensor> slots, double eps,
                        int64_t nq, int64_t nkv, int64_t d, int64_t T,
                        c10::optional<torch::Tensor> rot_freq);
void mul_sigmoid(torch::Tensor a, torch::Tensor gate_src, int64_t col0,
                 torch::Tensor y);
void silu_mul_halves(torch::Tensor gu, torch::Tensor y);
void hc_write_read(torch::Tensor xs, c10::optional<torch::Tensor> y,
                   c10::optional<torch::Tensor> mix,
                   c10::optional<torch::Tensor> w_out,
                   c10::optional<torch::Tensor> next_in,
                   c10::optional<torch::Tensor> next_wn,
                   c10::optional<torch::Tensor> out, double eps);
void gated_delta_scan(torch::Tensor qkv, torch::Tensor gates, int64_t b_col0,
                      int64_t a_col0, torch::Tensor a_log,
                      torch::Tensor dt_bias, torch::Tensor state,
                      torch::Tensor o, torch::Tensor pos,
                      c10::optional<torch::Tensor> lens,
                      c10::optional<torch::Tensor> slots, int64_t T,
                      int64_t H, int64_t KH, int64_t d, int64_t dv,
                      double unit_eps);
void latent_append(torch::Tensor src, int64_t col0, torch::Tensor wn,
                   double eps, int64_t R, torch::Tensor rot_freq,
                   torch::Tensor kcache, torch::Tensor pos,
                   c10::optional<torch::Tensor> lens,
                   c10::optional<torch::Tensor> slots, int64_t T);
void latent_q_pack(torch::Tensor q, torch::Tensor qabs, torch::Tensor rot_freq,
                   torch::Tensor pos, torch::Tensor out, int64_t T, int64_t H,
                   int64_t d);
void moe_up_act(torch::Tensor x, torch::Tensor w, torch::Tensor we,
                torch::Tensor act);
void moe_route(torch::Tensor logits, torch::Tensor we, int64_t top,
               double scale);
void moe_weighted_sum(torch::Tensor d, torch::Tensor we, torch::Tensor out);
}  // namespace dnet

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.doc() = "dnet_amd gfx950 (MI355X/CDNA4) kernels";
  m.def("rmsnorm", &dnet::rmsnorm, "fused RMSNorm (+residual)");
  m.def("gemv_bf16", &dnet::gemv_bf16, "bf16 decode GEMV");
  m.def("gemv_int8", &dnet::gemv_int8, "grouped-int8 W8A16 decode GEMV");
  m.def("attn_decode", &dnet::attn_decode, "GQA decode attention vs KV cache",
        py::arg("q"), py::arg("kcache"), py::arg("vcache"), py::arg("pos"),
        py::arg("out"), py::arg("scale"), py::arg("window"), py::arg("sinks"),
        py::arg("kscale"), py::arg("vscale"), py::arg("partials"),
        py::arg("splits"), py::arg("combine") = true);
  m.def("dequant_mxfp4", &dnet::dequant_mxfp4,
        "MXFP4 (e2m1 + e8m0 blocks) -> bf16");
  m.def("attn_prefill", &dnet::attn_prefill,
        "MFMA flash prefill attention (causal + window + sinks)",
        py::arg("q"), py::arg("k"), py::arg("v"), py::arg("sinks"),
        py::arg("out"), py::arg("q_off"), py::arg("window"),
        py::arg("scale"));
  m.def("attn_combine", &dnet::attn_combine,
        "merge split/rank flash-decode partials");
  m.def("rope_append", &dnet::rope_append, "fused RoPE + KV append (decode)",
        py::arg("q"), py::arg("k"), py::arg("v"), py::arg("kcache"),
        py::arg("vcache"), py::arg("pos"), py::arg("cos_table"),
        py::arg("sin_table"), py::arg("kscale"), py::arg("vscale"),
        py::arg("wpos") = c10::nullopt);
  m.def("swiglu", &dnet::swiglu, "fused SwiGLU");
  m.def("scratch_clean", &dnet::scratch_clean,
        "zero the split-k scratch region that plain combines left dirty");
  m.def("gemm_m16_will_defer", &dnet::gemm_m16_will_defer,
        "would gemm_m16(defer_combine=true) defer for this shape");
  m.def("rope_append_f32", &dnet::rope_append_f32,
        "RoPE+append reading+re-zeroing the qkv split-k f32 scratch");
  m.def("resid_add_f32", &dnet::resid_add_f32,
        "h += split-k f32 scratch (re-zeroed)");
  m.def("rmsnorm_f32", &dnet::rmsnorm_f32,
        "RMSNorm+residual reading+re-zeroing the split-k f32 scratch");
  m.def("swiglu_f32", &dnet::swiglu_f32,
        "SwiGLU reading+re-zeroing the split-k f32 scratch");
  m.def("dequant_int8", &dnet::dequant_int8, "grouped-int8 -> bf16 dequant");
  m.def("dequant_int4", &dnet::dequant_int4, "packed-int4 -> bf16 dequant");
  m.def("gemm_m16", &dnet::gemm_m16, "MFMA decode GEMM (M<=16, bf16 or int8)",
        py::arg("x"), py::arg("w"), py::arg("scales"), py::arg("bias"),
        py::arg("out"), py::arg("scratch"), py::arg("group"),
        py::arg("packed"), py::arg("bits"),
        py::arg("defer_combine") = false);
  m.def("moe_gateup", &dnet::moe_gateup,
        "grouped MoE gate+up GEMV with fused GLU and expert skip");
  m.def("moe_down", &dnet::moe_down,
        "grouped MoE down GEMV with weighted f32 accumulation");
  m.def("col_norm2", &dnet::col_norm2, "per-column L2 norms");
  m.def("gather_cols", &dnet::gather_cols, "pack kept columns");
  m.def("scatter_cols", &dnet::scatter_cols, "zero + scatter kept columns");
  m.def("rmsnorm_rows", &dnet::rmsnorm_rows,
        "RMSNorm with fp32 statistics, fp32/bf16 in and out");
  m.def("ls_resid_rmsnorm", &dnet::ls_resid_rmsnorm,
        "fp32 residual += layer-scaled branches, fused with the next norm");
  m.def("xielu", &dnet::xielu, "two-parameter squared/exponential unit");
  m.def("qknorm_append", &dnet::qknorm_append,
        "q/k RMSNorm (whole projection or per head) + KV append");
  m.def("attn_mod", &dnet::attn_mod,
        "score-modified causal attention (decode + ragged prefill), optional "
        "window with pooled blocks");
  m.def("resid_branches_rmsnorm", &dnet::resid_branches_rmsnorm,
        "fp32 residual += normalized/plain branches, fused with the next "
        "norm and a cast copy");
  m.def("gated_group_rmsnorm", &dnet::gated_group_rmsnorm,
        "grouped RMSNorm with a silu/sigmoid gate before or after");
  m.def("act_slice", &dnet::act_slice,
        "unary activation of a column range (relu^2, tanh)");
  m.def("gelu_gather_mul", &dnet::gelu_gather_mul,
        "gelu_tanh(z) * table[token, col0:col0+n]");
  m.def("clamped_glu", &dnet::clamped_glu, "clamped GLU of [gate | up]");
  m.def("kv_pool_update", &dnet::kv_pool_update,
        "block means of the KV cache for the blocks a step completes");
  m.def("causal_conv_silu", &dnet::causal_conv_silu,
        "per-channel causal convolution + SiLU with a per-slot tail state");
  m.def("ssd_scan", &dnet::ssd_scan,
        "selective state-space recurrence (scalar decay per head)");
  m.def("delta_scan", &dnet::delta_scan, "generalized delta-rule recurrence");
  m.def("hc_write_read", &dnet::hc_write_read,
        "residual streams: write a sublayer's result, read the next input");
  m.def("pair_hash_embed", &dnet::pair_hash_embed,
        "token embedding + hashed (previous, current) pair embedding");
  m.def("causal_conv_residual", &dnet::causal_conv_residual,
        "x + causal per-channel convolution of the fp32 residual");
  m.def("decay_scan", &dnet::decay_scan,
        "linear attention with a constant decay per head");
  m.def("qknorm_half_append", &dnet::qknorm_half_append,
        "whole-projection q/k norm, half-split rotation, cache append");
  m.def("mul_sigmoid", &dnet::mul_sigmoid, "a * sigmoid(gate columns)");
  m.def("silu_mul_halves", &dnet::silu_mul_halves,
        "silu(gate half) * up half, any dtype and width");
  m.def("gated_delta_scan", &dnet::gated_delta_scan,
        "gated delta-rule recurrence");
  m.def("latent_append", &dnet::latent_append,
        "latent attention: norm + rotation + cache append of the shared row");
  m.def("latent_q_pack", &dnet::latent_q_pack,
        "latent attention: queries in the cache row's layout");
  m.def("moe_up_act", &dnet::moe_up_act,
        "grouped ungated expert up projection + squared ReLU");
  m.def("moe_route", &dnet::moe_route,
        "softmax over all experts, top-k kept, scaled, not renormalized");
  m.def("moe_weighted_sum", &dnet::moe_weighted_sum,
        "sum over experts of routing weight times expert result");
}
