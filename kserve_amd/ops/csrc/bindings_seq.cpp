// Python bindings for the sequence-mixer kernels that keep a 32-bit residual
// stream and recurrent state (state-space scan, causal convolution, fp32
// paged attention, grouped/offset RMS norms, clamped GLU). A module of its
// own so that a model built from these mechanisms compiles nothing else.
#include "bindings_common.h"

extern "C" {
hipError_t ks_embed_scale_sinpos(void*, const void*, const void*, const void*,
                                 const void*, float, int, int, int,
                                 hipStream_t);
hipError_t ks_add_rms_norm_f32res(void*, const void*, long, float, const void*,
                                  long, float, const void*, float, float,
                                  void*, int, int, int, hipStream_t);
hipError_t ks_gated_group_rms_norm(void*, const void*, const void*, long,
                                   const void*, float, int, int, int, int,
                                   hipStream_t);
hipError_t ks_causal_conv_silu(void*, const void*, long, const void*,
                               const void*, void*, const void*, const void*,
                               const void*, const void*, int, int, int, int,
                               int, hipStream_t);
hipError_t ks_ssd_scan(void*, const void*, const void*, long, int, const void*,
                       const void*, const void*, void*, const void*,
                       const void*, const void*, int, int, int, int, int,
                       hipStream_t);
hipError_t ks_qk_norm_temp_cache(void*, const void*, const void*, const void*,
                                 long, const void*, const void*, const void*,
                                 const void*, void*, void*, float, float, int,
                                 int, int, int, int, int, int, int,
                                 hipStream_t);
hipError_t ks_ctx_attention_f32(void*, const void*, const void*, const void*,
                                const void*, int, const void*, const void*,
                                const void*, long, float, int, int, int, int,
                                int, int, int, int, hipStream_t);
hipError_t ks_clamped_swiglu(void*, const void*, int, int, float, float, int,
                             hipStream_t);
}

namespace {

// activation dtype of a call: fp32 or bf16, nothing else
int act_is_f32(const at::Tensor& t, const char* name) {
  TORCH_CHECK(t.is_cuda(), name, " must be on GPU");
  TORCH_CHECK(t.scalar_type() == at::kFloat || t.scalar_type() == at::kBFloat16,
              name, " must be fp32 or bf16");
  return t.scalar_type() == at::kFloat;
}

#define CHECK_F32(t)                                                     \
  TORCH_CHECK((t).is_cuda() && (t).scalar_type() == at::kFloat &&        \
                  (t).is_contiguous(),                                   \
              #t " must be a contiguous fp32 GPU tensor")
#define CHECK_I32(t)                                                     \
  TORCH_CHECK((t).is_cuda() && (t).scalar_type() == at::kInt &&          \
                  (t).is_contiguous(),                                   \
              #t " must be a contiguous int32 GPU tensor")
#define CHECK_I64(t)                                                     \
  TORCH_CHECK((t).is_cuda() && (t).scalar_type() == at::kLong &&         \
                  (t).is_contiguous(),                                   \
              #t " must be a contiguous int64 GPU tensor")
// 2-D view whose rows may be strided (a column slice of a projection)
#define CHECK_ROWS(t)                                                    \
  TORCH_CHECK((t).dim() == 2 && (t).stride(1) == 1, #t " rows must be dense")

void embed_scale_sinpos(at::Tensor& out, at::Tensor& table, at::Tensor& tokens,
                        at::Tensor& positions, at::Tensor& inv_freq,
                        double scale) {
  CHECK_F32(out);
  CHECK_F32(inv_freq);
  CHECK_I64(tokens);
  CHECK_I64(positions);
  TORCH_CHECK(table.is_contiguous() && table.dim() == 2, "table [vocab, width]");
  const int width = table.size(1), rows = tokens.numel();
  TORCH_CHECK(out.numel() == (int64_t)rows * width &&
                  positions.numel() == rows && inv_freq.numel() * 2 >= width,
              "embed_scale_sinpos: shape mismatch");
  check_hip(ks_embed_scale_sinpos(out.data_ptr(), table.data_ptr(),
                                  tokens.data_ptr(), positions.data_ptr(),
                                  inv_freq.data_ptr(), (float)scale, rows,
                                  width, act_is_f32(table, "table"),
                                  current_stream()),
            "embed_scale_sinpos");
}

void add_rms_norm_f32res(at::Tensor& residual,
                         const c10::optional<at::Tensor>& d0, double s0,
                         const c10::optional<at::Tensor>& d1, double s1,
                         at::Tensor& weight, double w_offset, double eps,
                         at::Tensor& out) {
  CHECK_F32(residual);
  CHECK_F32(weight);
  TORCH_CHECK(residual.dim() == 2 && out.is_contiguous(), "residual [T, W]");
  const int rows = residual.size(0), width = residual.size(1);
  TORCH_CHECK(weight.numel() == width && out.numel() == residual.numel(),
              "add_rms_norm_f32res: shape mismatch");
  const int f32 = act_is_f32(out, "out");
  const void *p0 = nullptr, *p1 = nullptr;
  long st0 = 0, st1 = 0;
  if (d0.has_value()) {
    CHECK_ROWS(*d0);
    TORCH_CHECK(act_is_f32(*d0, "d0") == f32 && d0->size(0) == rows &&
                    d0->size(1) == width,
                "d0: dtype/shape mismatch");
    p0 = d0->data_ptr();
    st0 = d0->stride(0);
  }
  if (d1.has_value()) {
    CHECK_ROWS(*d1);
    TORCH_CHECK(act_is_f32(*d1, "d1") == f32 && d1->size(0) == rows &&
                    d1->size(1) == width,
                "d1: dtype/shape mismatch");
    p1 = d1->data_ptr();
    st1 = d1->stride(0);
  }
  check_hip(ks_add_rms_norm_f32res(residual.data_ptr(), p0, st0, (float)s0, p1,
                                   st1, (float)s1, weight.data_ptr(),
                                   (float)w_offset, (float)eps, out.data_ptr(),
                                   rows, width, f32, current_stream()),
            "add_rms_norm_f32res");
}

void gated_group_rms_norm(at::Tensor& out, at::Tensor& y, at::Tensor& z,
                          at::Tensor& weight, double eps, int64_t groups) {
  CHECK_F32(y);
  CHECK_F32(weight);
  CHECK_ROWS(z);
  TORCH_CHECK(y.dim() == 2 && out.is_contiguous(), "y [T, inner]");
  const int rows = y.size(0), inner = y.size(1);
  const int f32 = act_is_f32(out, "out");
  TORCH_CHECK(act_is_f32(z, "z") == f32 && z.size(0) == rows &&
                  z.size(1) == inner && weight.numel() == inner &&
                  out.numel() == y.numel() && groups > 0 &&
                  inner % groups == 0,
              "gated_group_rms_norm: dtype/shape mismatch");
  check_hip(ks_gated_group_rms_norm(out.data_ptr(), y.data_ptr(), z.data_ptr(),
                                    z.stride(0), weight.data_ptr(), (float)eps,
                                    rows, inner, (int)groups, f32,
                                    current_stream()),
            "gated_group_rms_norm");
}

void causal_conv_silu(at::Tensor& out, at::Tensor& in, at::Tensor& w,
                      at::Tensor& bias, at::Tensor& conv_state,
                      at::Tensor& positions, at::Tensor& seq_of_token,
                      at::Tensor& cu_seqlens, at::Tensor& slots) {
  CHECK_F32(out);
  CHECK_F32(w);
  CHECK_F32(bias);
  CHECK_ROWS(in);
  CHECK_I64(positions);
  CHECK_I32(seq_of_token);
  CHECK_I32(cu_seqlens);
  CHECK_I32(slots);
  const int tokens = in.size(0), channels = in.size(1);
  const int taps = w.size(1), num_seqs = slots.numel();
  const int f32 = act_is_f32(in, "in");
  TORCH_CHECK(w.dim() == 2 && w.size(0) == channels &&
                  bias.numel() == channels &&
                  out.numel() == (int64_t)tokens * channels &&
                  positions.numel() >= tokens &&
                  seq_of_token.numel() >= tokens &&
                  cu_seqlens.numel() == num_seqs + 1,
              "causal_conv_silu: shape mismatch");
  TORCH_CHECK(conv_state.is_contiguous() && conv_state.dim() == 3 &&
                  act_is_f32(conv_state, "conv_state") == f32 &&
                  conv_state.size(1) == std::max(taps - 1, 1) &&
                  conv_state.size(2) == channels,
              "conv_state must be [slots, taps-1, channels] in the input dtype");
  check_hip(ks_causal_conv_silu(out.data_ptr(), in.data_ptr(), in.stride(0),
                                w.data_ptr(), bias.data_ptr(),
                                conv_state.data_ptr(), positions.data_ptr(),
                                seq_of_token.data_ptr(), cu_seqlens.data_ptr(),
                                slots.data_ptr(), tokens, num_seqs, channels,
                                taps, f32, current_stream()),
            "causal_conv_silu");
}

void ssd_scan(at::Tensor& y, at::Tensor& xbc, at::Tensor& dt_raw,
              at::Tensor& dt_bias, at::Tensor& a_log, at::Tensor& d_skip,
              at::Tensor& state, at::Tensor& positions, at::Tensor& cu_seqlens,
              at::Tensor& slots, int64_t groups) {
  CHECK_F32(y);
  CHECK_F32(xbc);
  CHECK_F32(dt_bias);
  CHECK_F32(a_log);
  CHECK_F32(d_skip);
  CHECK_F32(state);
  CHECK_ROWS(dt_raw);
  CHECK_I64(positions);
  CHECK_I32(cu_seqlens);
  CHECK_I32(slots);
  TORCH_CHECK(state.dim() == 4, "state [slots, heads, P, N]");
  const int heads = state.size(1), P = state.size(2), N = state.size(3);
  const int tokens = xbc.size(0), num_seqs = slots.numel();
  TORCH_CHECK(xbc.dim() == 2 &&
                  xbc.size(1) == heads * P + 2 * groups * N &&
                  y.numel() == (int64_t)tokens * heads * P &&
                  dt_raw.size(0) == tokens && dt_raw.size(1) == heads &&
                  dt_bias.numel() == heads && a_log.numel() == heads &&
                  d_skip.numel() == heads && positions.numel() >= tokens &&
                  cu_seqlens.numel() == num_seqs + 1,
              "ssd_scan: shape mismatch");
  check_hip(ks_ssd_scan(y.data_ptr(), xbc.data_ptr(), dt_raw.data_ptr(),
                        dt_raw.stride(0), act_is_f32(dt_raw, "dt_raw"),
                        dt_bias.data_ptr(), a_log.data_ptr(),
                        d_skip.data_ptr(), state.data_ptr(),
                        positions.data_ptr(), cu_seqlens.data_ptr(),
                        slots.data_ptr(), num_seqs, heads, (int)groups, P, N,
                        current_stream()),
            "ssd_scan");
}

void qk_norm_temp_cache(at::Tensor& q_out, at::Tensor& q, at::Tensor& k,
                        at::Tensor& v, at::Tensor& qw, at::Tensor& kw,
                        at::Tensor& positions, at::Tensor& slot_mapping,
                        at::Tensor& k_cache, at::Tensor& v_cache, double eps,
                        double temp_coef, int64_t temp_every, int64_t heads) {
  CHECK_F32(q_out);
  CHECK_F32(qw);
  CHECK_F32(kw);
  CHECK_ROWS(q);
  CHECK_ROWS(k);
  CHECK_ROWS(v);
  CHECK_I64(positions);
  CHECK_I32(slot_mapping);
  TORCH_CHECK(k_cache.dim() == 4 && v_cache.dim() == 4 &&
                  k_cache.is_contiguous() && v_cache.is_contiguous(),
              "caches [blocks, kv_heads, block, dim]");
  const int f32 = act_is_f32(q, "q");
  const int tokens = q.size(0);
  const int G = k_cache.size(1), bs = k_cache.size(2), D = k_cache.size(3);
  const int DV = v_cache.size(3);
  TORCH_CHECK(act_is_f32(k, "k") == f32 && act_is_f32(v, "v") == f32 &&
                  act_is_f32(k_cache, "k_cache") == f32 &&
                  act_is_f32(v_cache, "v_cache") == f32,
              "qk_norm_temp_cache: dtype mismatch");
  TORCH_CHECK(q.size(1) == heads * D && k.size(1) == G * D &&
                  v.size(1) == G * DV && k.size(0) == tokens &&
                  v.size(0) == tokens && q.stride(0) == k.stride(0) &&
                  q.stride(0) == v.stride(0) && qw.numel() == heads * D &&
                  kw.numel() == G * D && v_cache.size(1) == G &&
                  v_cache.size(2) == bs && v_cache.size(0) == k_cache.size(0) &&
                  q_out.numel() == (int64_t)tokens * heads * D &&
                  positions.numel() >= tokens && slot_mapping.numel() >= tokens,
              "qk_norm_temp_cache: shape mismatch");
  check_hip(ks_qk_norm_temp_cache(
                q_out.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(),
                q.stride(0), qw.data_ptr(), kw.data_ptr(),
                positions.data_ptr(), slot_mapping.data_ptr(),
                k_cache.data_ptr(), v_cache.data_ptr(), (float)eps,
                (float)temp_coef, (int)temp_every, tokens, (int)heads, G, D,
                DV, bs, f32, current_stream()),
            "qk_norm_temp_cache");
}

void ctx_attention_f32(at::Tensor& out, at::Tensor& q, at::Tensor& k_cache,
                       at::Tensor& v_cache, at::Tensor& block_tables,
                       at::Tensor& cu_q, at::Tensor& ctx_lens,
                       const c10::optional<at::Tensor>& gate, double scale,
                       int64_t max_q_len, int64_t heads) {
  CHECK_F32(q);
  CHECK_I32(cu_q);
  CHECK_I32(ctx_lens);
  TORCH_CHECK(block_tables.is_cuda() && block_tables.scalar_type() == at::kInt &&
                  block_tables.dim() == 2 && block_tables.stride(1) == 1,
              "block_tables [seqs, blocks] int32");
  TORCH_CHECK(k_cache.dim() == 4 && v_cache.dim() == 4 &&
                  k_cache.is_contiguous() && v_cache.is_contiguous() &&
                  out.is_contiguous(),
              "caches [blocks, kv_heads, block, dim]");
  const int f32 = act_is_f32(out, "out");
  const int G = k_cache.size(1), bs = k_cache.size(2), D = k_cache.size(3);
  const int DV = v_cache.size(3);
  const int num_seqs = ctx_lens.numel();
  const int64_t tokens = q.numel() / (heads * D);
  TORCH_CHECK(act_is_f32(k_cache, "k_cache") == f32 &&
                  act_is_f32(v_cache, "v_cache") == f32 &&
                  q.numel() == tokens * heads * D &&
                  out.numel() == tokens * heads * DV &&
                  cu_q.numel() == num_seqs + 1 &&
                  block_tables.size(0) >= num_seqs && v_cache.size(1) == G &&
                  v_cache.size(2) == bs,
              "ctx_attention_f32: dtype/shape mismatch");
  const void* gp = nullptr;
  long gst = 0;
  if (gate.has_value()) {
    CHECK_ROWS(*gate);
    TORCH_CHECK(act_is_f32(*gate, "gate") == f32 && gate->size(0) == tokens &&
                    gate->size(1) == heads,
                "gate [T, heads] in the activation dtype");
    gp = gate->data_ptr();
    gst = gate->stride(0);
  }
  check_hip(ks_ctx_attention_f32(
                out.data_ptr(), q.data_ptr(), k_cache.data_ptr(),
                v_cache.data_ptr(), block_tables.data_ptr(),
                (int)block_tables.stride(0), cu_q.data_ptr(),
                ctx_lens.data_ptr(), gp, gst, (float)scale, num_seqs,
                (int)max_q_len, (int)heads, G, D, DV, bs, f32,
                current_stream()),
            "ctx_attention_f32");
}

void clamped_swiglu(at::Tensor& out, at::Tensor& input, double alpha,
                    double limit) {
  TORCH_CHECK(input.is_contiguous() && out.is_contiguous(), "contiguous");
  const int d = input.size(-1) / 2;
  const int rows = input.numel() / (2 * d);
  const int f32 = act_is_f32(input, "input");
  TORCH_CHECK(act_is_f32(out, "out") == f32 &&
                  out.numel() == (int64_t)rows * d && input.size(-1) == 2 * d,
              "clamped_swiglu: dtype/shape mismatch");
  check_hip(ks_clamped_swiglu(out.data_ptr(), input.data_ptr(), rows, d,
                              (float)alpha, (float)limit, f32,
                              current_stream()),
            "clamped_swiglu");
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.def("embed_scale_sinpos", &embed_scale_sinpos,
        "scaled embedding + interleaved sinusoidal positions (fp32 out)");
  m.def("add_rms_norm_f32res", &add_rms_norm_f32res,
        "fp32 residual += scaled deltas, then offset-weight RMS norm");
  m.def("gated_group_rms_norm", &gated_group_rms_norm,
        "y * silu(z), RMS norm per group, times weight");
  m.def("causal_conv_silu", &causal_conv_silu,
        "varlen depthwise causal conv + silu with per-slot history");
  m.def("ssd_scan", &ssd_scan, "state-space scan with per-slot fp32 state");
  m.def("qk_norm_temp_cache", &qk_norm_temp_cache,
        "whole-projection q/k RMS norm, query temperature, KV page scatter");
  m.def("ctx_attention_f32", &ctx_attention_f32,
        "paged causal attention, fp32 scores/weights, optional output gate");
  m.def("clamped_swiglu", &clamped_swiglu, "clamped GLU activation");
  def_sampling(m);
}
