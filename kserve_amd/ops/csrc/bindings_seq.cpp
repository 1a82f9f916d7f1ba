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
                                  void*, int, int, int, int, hipStream_t);
hipError_t ks_gated_group_rms_norm(void*, const void*, const void*, long,
                                   const void*, int, float, int, int, int, int,
                                   int, hipStream_t);
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
                                int, int, int, int, const void*, int,
                                const void*, int, long, void*, int,
                                hipStream_t);
int ks_ctx_attention_decode_splits(int, int, int, int, int);
hipError_t ks_qk_headnorm_rope_cache(void*, const void*, const void*,
                                     const void*, long, const void*,
                                     const void*, const void*, const void*,
                                     void*, void*, float, int, int, int, int,
                                     int, int, const void*, int, int,
                                     const void*, int, int, hipStream_t);
hipError_t ks_post_norm_add_rms_norm(void*, const void*, long, int, float,
                                     const void*, const void*, const void*,
                                     float, float, void*, int, int, int,
                                     hipStream_t);
hipError_t ks_router_topk(void*, void*, void*, const void*, int, int, int, int,
                          int, const void*, float, float, hipStream_t);
hipError_t ks_route_tokens(void*, void*, void*, void*, const void*, long,
                           const void*, int, int, int, int, int, int,
                           const void*, float, float, int, hipStream_t);
hipError_t ks_gather_scale_rows(void*, const void*, long, const void*,
                                const void*, int, int, int, hipStream_t);
hipError_t ks_combine_rows(void*, const void*, const void*, int, const void*,
                           long, int, int, int, const void*, const void*, long,
                           const void*, hipStream_t);
hipError_t ks_post_layer_norm_add(void*, const void*, long, int, const void*,
                                  float, float, void*, int, const void*, int,
                                  int, hipStream_t);
hipError_t ks_latent_norm_rope_cache(void*, const void*, long, int, int, int,
                                     int, const void*, const void*,
                                     const void*, const void*, void*, float,
                                     const void*, int, int, hipStream_t);
hipError_t ks_head_matmul_rope(void*, const void*, long, const void*, int, int,
                               int, int, int, const void*, const void*, int,
                               int, int, hipStream_t);
hipError_t ks_glu_silu_scale(void*, const void*, const void*, int, int, int,
                             hipStream_t);
hipError_t ks_bias_gelu_tanh(void*, const void*, const void*, int, int, int,
                             hipStream_t);
hipError_t ks_clamped_swiglu(void*, const void*, int, int, float, float, int,
                             hipStream_t);
hipError_t ks_relu2_scale(void*, const void*, const void*, int, int, int,
                          hipStream_t);
hipError_t ks_scale_softcap(void*, const void*, float, float, long, int,
                            hipStream_t);
hipError_t ks_rope_scale_heads(void*, const void*, long, const void*,
                               const void*, int, int, int, float, int, float,
                               int, int, int, hipStream_t);
hipError_t ks_unit_norm_heads(void*, long, int, int, float, int, float, int,
                              float, hipStream_t);
hipError_t ks_linear_scan(void*, const void*, long, const void*, long,
                          const void*, long, const void*, const void*,
                          const void*, long, int, const void*, const void*,
                          void*, const void*, const void*, const void*, int,
                          int, int, int, int, hipStream_t);
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
                        at::Tensor& positions,
                        const c10::optional<at::Tensor>& inv_freq_opt,
                        double scale) {
  CHECK_F32(out);
  const void* inv_freq_ptr = nullptr;
  int64_t n_freq = 1 << 30;
  if (inv_freq_opt.has_value()) {
    const at::Tensor& inv_freq = *inv_freq_opt;
    CHECK_F32(inv_freq);
    inv_freq_ptr = inv_freq.data_ptr();
    n_freq = inv_freq.numel();
  }
  CHECK_I64(tokens);
  CHECK_I64(positions);
  TORCH_CHECK(table.is_contiguous() && table.dim() == 2, "table [vocab, width]");
  const int width = table.size(1), rows = tokens.numel();
  TORCH_CHECK(out.numel() == (int64_t)rows * width &&
                  positions.numel() == rows && n_freq * 2 >= width,
              "embed_scale_sinpos: shape mismatch");
  check_hip(ks_embed_scale_sinpos(out.data_ptr(), table.data_ptr(),
                                  tokens.data_ptr(), positions.data_ptr(),
                                  inv_freq_ptr, (float)scale, rows,
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
  // the deltas share a dtype: the output's, or fp32 beside a bf16 output
  int df32 = f32;
  if (d0.has_value()) df32 = act_is_f32(*d0, "d0");
  else if (d1.has_value()) df32 = act_is_f32(*d1, "d1");
  TORCH_CHECK(df32 == f32 || df32 == 1, "bf16 deltas need a bf16 output");
  const void *p0 = nullptr, *p1 = nullptr;
  long st0 = 0, st1 = 0;
  if (d0.has_value()) {
    CHECK_ROWS(*d0);
    TORCH_CHECK(act_is_f32(*d0, "d0") == df32 && d0->size(0) == rows &&
                    d0->size(1) == width,
                "d0: dtype/shape mismatch");
    p0 = d0->data_ptr();
    st0 = d0->stride(0);
  }
  if (d1.has_value()) {
    CHECK_ROWS(*d1);
    TORCH_CHECK(act_is_f32(*d1, "d1") == df32 && d1->size(0) == rows &&
                    d1->size(1) == width,
                "d1: dtype/shape mismatch");
    p1 = d1->data_ptr();
    st1 = d1->stride(0);
  }
  check_hip(ks_add_rms_norm_f32res(residual.data_ptr(), p0, st0, (float)s0, p1,
                                   st1, (float)s1, weight.data_ptr(),
                                   (float)w_offset, (float)eps, out.data_ptr(),
                                   rows, width, f32, df32, current_stream()),
            "add_rms_norm_f32res");
}

void gated_group_rms_norm(at::Tensor& out, at::Tensor& y, at::Tensor& z,
                          const c10::optional<at::Tensor>& weight_opt,
                          double eps, int64_t groups, bool gate_after) {
  CHECK_F32(y);
  const void* wp = nullptr;
  int64_t wn = y.size(1);
  if (weight_opt.has_value()) {
    CHECK_F32(*weight_opt);
    wp = weight_opt->data_ptr();
    wn = weight_opt->numel();
  }
  CHECK_ROWS(z);
  TORCH_CHECK(y.dim() == 2 && out.is_contiguous(), "y [T, inner]");
  const int rows = y.size(0), inner = y.size(1);
  const int f32 = act_is_f32(out, "out");
  TORCH_CHECK(act_is_f32(z, "z") == f32 && z.size(0) == rows &&
                  z.size(1) == inner && wn > 0 && inner % wn == 0 &&
                  out.numel() == y.numel() && groups > 0 &&
                  inner % groups == 0,
              "gated_group_rms_norm: dtype/shape mismatch");
  check_hip(ks_gated_group_rms_norm(out.data_ptr(), y.data_ptr(), z.data_ptr(),
                                    z.stride(0), wp, (int)wn, (float)eps, rows,
                                    inner, (int)groups, gate_after ? 1 : 0,
                                    f32, current_stream()),
            "gated_group_rms_norm");
}

void causal_conv_silu(at::Tensor& out, at::Tensor& in, at::Tensor& w,
                      const c10::optional<at::Tensor>& bias_opt,
                      at::Tensor& conv_state,
                      at::Tensor& positions, at::Tensor& seq_of_token,
                      at::Tensor& cu_seqlens, at::Tensor& slots) {
  CHECK_F32(out);
  CHECK_F32(w);
  const void* bias_ptr = nullptr;
  if (bias_opt.has_value()) {
    CHECK_F32(*bias_opt);
    TORCH_CHECK(bias_opt->numel() == in.size(1), "bias [channels]");
    bias_ptr = bias_opt->data_ptr();
  }
  CHECK_ROWS(in);
  CHECK_I64(positions);
  CHECK_I32(seq_of_token);
  CHECK_I32(cu_seqlens);
  CHECK_I32(slots);
  const int tokens = in.size(0), channels = in.size(1);
  const int taps = w.size(1), num_seqs = slots.numel();
  const int f32 = act_is_f32(in, "in");
  TORCH_CHECK(w.dim() == 2 && w.size(0) == channels &&
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
                                w.data_ptr(), bias_ptr,
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
                       int64_t max_q_len, int64_t heads,
                       const c10::optional<at::Tensor>& sink, int64_t chunk,
                       const c10::optional<at::Tensor>& out_inv_freq,
                       int64_t window) {
  CHECK_F32(q);
  CHECK_I32(cu_q);
  CHECK_I32(ctx_lens);
  TORCH_CHECK(block_tables.is_cuda() && block_tables.scalar_type() == at::kInt &&
                  block_tables.dim() == 2 && block_tables.stride(1) == 1,
              "block_tables [seqs, blocks] int32");
  TORCH_CHECK(k_cache.dim() == 4 && v_cache.dim() == 4 &&
                  k_cache.is_contiguous() && out.is_contiguous(),
              "caches [blocks, kv_heads, block, dim]");
  const int f32 = act_is_f32(out, "out");
  const int G = k_cache.size(1), bs = k_cache.size(2), D = k_cache.size(3);
  const int DV = v_cache.size(3);
  // the values may be a column range of wider rows (a view of the key pool)
  const int64_t vrs = v_cache.stride(2);
  TORCH_CHECK(v_cache.stride(3) == 1 && vrs >= DV &&
                  v_cache.stride(1) == vrs * bs &&
                  v_cache.stride(0) == vrs * bs * G,
              "v_cache: dense pages of rows with one common stride");
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
  const void *sp = nullptr, *fp = nullptr;
  if (sink.has_value()) {
    CHECK_F32(*sink);
    TORCH_CHECK(sink->numel() == heads, "sink [heads] fp32");
    sp = sink->data_ptr();
  }
  if (out_inv_freq.has_value()) {
    CHECK_F32(*out_inv_freq);
    TORCH_CHECK(DV % 2 == 0 && out_inv_freq->numel() == DV / 2,
                "out_inv_freq [vdim / 2] fp32");
    fp = out_inv_freq->data_ptr();
  }
  TORCH_CHECK(chunk >= 0 && window >= 0 && !(chunk > 0 && window > 0),
              "chunk / window: not negative, at most one of them");
  // a decode batch splits every sequence's keys over several blocks, which
  // leave partial results in a scratch tensor for a merge pass
  int nsplit = 1;
  at::Tensor ws;
  if (max_q_len == 1) {
    nsplit = ks_ctx_attention_decode_splits(num_seqs, (int)heads, G,
                                            (int)window, fp != nullptr);
    if (nsplit > 1)
      ws = at::empty({(int64_t)num_seqs * heads * nsplit * (DV + 2)},
                     q.options().dtype(at::kFloat));
  }
  check_hip(ks_ctx_attention_f32(
                out.data_ptr(), q.data_ptr(), k_cache.data_ptr(),
                v_cache.data_ptr(), block_tables.data_ptr(),
                (int)block_tables.stride(0), cu_q.data_ptr(),
                ctx_lens.data_ptr(), gp, gst, (float)scale, num_seqs,
                (int)max_q_len, (int)heads, G, D, DV, bs, f32, sp, (int)chunk,
                fp, (int)window, (long)vrs,
                nsplit > 1 ? ws.data_ptr() : nullptr, nsplit,
                current_stream()),
            "ctx_attention_f32");
}

void qk_headnorm_rope_cache(at::Tensor& q_out, at::Tensor& q, at::Tensor& k,
                            at::Tensor& v,
                            const c10::optional<at::Tensor>& qw_opt,
                            const c10::optional<at::Tensor>& kw_opt,
                            at::Tensor& positions, at::Tensor& slot_mapping,
                            at::Tensor& k_cache, at::Tensor& v_cache,
                            double eps, int64_t heads,
                            const c10::optional<at::Tensor>& qk_inv_freq,
                            bool v_unit_norm,
                            const c10::optional<at::Tensor>& v_inv_freq) {
  CHECK_F32(q_out);
  // without weights the norm is plain x / rms(x)
  const void *qwp = nullptr, *kwp = nullptr;
  if (qw_opt.has_value()) {
    CHECK_F32(*qw_opt);
    TORCH_CHECK(qw_opt->numel() == k_cache.size(3), "qw [dim]");
    qwp = qw_opt->data_ptr();
  }
  if (kw_opt.has_value()) {
    CHECK_F32(*kw_opt);
    TORCH_CHECK(kw_opt->numel() == k_cache.size(3), "kw [dim]");
    kwp = kw_opt->data_ptr();
  }
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
              "qk_headnorm_rope_cache: dtype mismatch");
  TORCH_CHECK(q.size(1) == heads * D && k.size(1) == G * D &&
                  v.size(1) == G * DV && k.size(0) == tokens &&
                  v.size(0) == tokens && q.stride(0) == k.stride(0) &&
                  q.stride(0) == v.stride(0) && v_cache.size(1) == G &&
                  v_cache.size(2) == bs && v_cache.size(0) == k_cache.size(0) &&
                  q_out.numel() == (int64_t)tokens * heads * D &&
                  positions.numel() >= tokens && slot_mapping.numel() >= tokens,
              "qk_headnorm_rope_cache: shape mismatch");
  const void *qf = nullptr, *vf = nullptr;
  int qh = 0, vh = 0;
  if (qk_inv_freq.has_value()) {
    CHECK_F32(*qk_inv_freq);
    qh = qk_inv_freq->numel();
    TORCH_CHECK(2 * qh <= D, "more rotated coordinates than the head has");
    qf = qk_inv_freq->data_ptr();
  }
  if (v_inv_freq.has_value()) {
    CHECK_F32(*v_inv_freq);
    vh = v_inv_freq->numel();
    TORCH_CHECK(2 * vh <= DV, "more rotated coordinates than the value has");
    vf = v_inv_freq->data_ptr();
  }
  check_hip(ks_qk_headnorm_rope_cache(
                q_out.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(),
                q.stride(0), qwp, kwp,
                positions.data_ptr(), slot_mapping.data_ptr(),
                k_cache.data_ptr(), v_cache.data_ptr(), (float)eps, tokens,
                (int)heads, G, D, DV, bs, qf, qh, v_unit_norm ? 1 : 0, vf, vh,
                f32, current_stream()),
            "qk_headnorm_rope_cache");
}

void post_norm_add_rms_norm(at::Tensor& residual,
                            const c10::optional<at::Tensor>& delta,
                            double post_gain,
                            const c10::optional<at::Tensor>& layer_scale,
                            double eps, double next_gain,
                            const c10::optional<at::Tensor>& out,
                            const c10::optional<at::Tensor>& add_rows,
                            const c10::optional<at::Tensor>& add_vec) {
  CHECK_F32(residual);
  TORCH_CHECK(residual.dim() == 2, "residual [T, W]");
  const int rows = residual.size(0), width = residual.size(1);
  const void *dp = nullptr, *lp = nullptr, *rp = nullptr, *vp = nullptr;
  void* op = nullptr;
  long dst = 0;
  int d_f32 = 1, o_f32 = 1;
  if (delta.has_value()) {
    CHECK_ROWS(*delta);
    TORCH_CHECK(layer_scale.has_value(), "delta needs a layer scale");
    CHECK_F32(*layer_scale);
    TORCH_CHECK(delta->size(0) == rows && delta->size(1) == width &&
                    layer_scale->numel() == width,
                "delta / layer_scale: shape mismatch");
    d_f32 = act_is_f32(*delta, "delta");
    dp = delta->data_ptr();
    dst = delta->stride(0);
    lp = layer_scale->data_ptr();
  }
  if (add_rows.has_value()) {
    CHECK_F32(*add_rows);
    TORCH_CHECK(add_rows->numel() == residual.numel(), "add_rows [T, W]");
    rp = add_rows->data_ptr();
  }
  if (add_vec.has_value()) {
    CHECK_F32(*add_vec);
    TORCH_CHECK(add_vec->numel() == width, "add_vec [W]");
    vp = add_vec->data_ptr();
  }
  if (out.has_value()) {
    TORCH_CHECK(out->is_contiguous() && out->numel() == residual.numel(),
                "out [T, W]");
    o_f32 = act_is_f32(*out, "out");
    op = out->data_ptr();
  }
  check_hip(ks_post_norm_add_rms_norm(residual.data_ptr(), dp, dst, d_f32,
                                      (float)post_gain, lp, rp, vp, (float)eps,
                                      (float)next_gain, op, o_f32, rows, width,
                                      current_stream()),
            "post_norm_add_rms_norm");
}

void router_topk(at::Tensor& idx, at::Tensor& w,
                 const c10::optional<at::Tensor>& dense, at::Tensor& logits,
                 bool softmax, bool renorm,
                 const c10::optional<at::Tensor>& correction,
                 double renorm_eps, double weight_scale) {
  CHECK_F32(logits);
  CHECK_F32(w);
  CHECK_I32(idx);
  TORCH_CHECK(logits.dim() == 2 && idx.dim() == 2, "logits [T, E], idx [T, top]");
  const int T = logits.size(0), E = logits.size(1), top = idx.size(1);
  TORCH_CHECK(idx.size(0) == T && w.numel() == idx.numel(),
              "router_topk: shape mismatch");
  void* dp = nullptr;
  if (dense.has_value()) {
    CHECK_F32(*dense);
    TORCH_CHECK(dense->numel() == logits.numel(), "dense [T, E]");
    dp = dense->data_ptr();
  }
  const void* cp = nullptr;
  if (correction.has_value()) {
    CHECK_F32(*correction);
    TORCH_CHECK(correction->numel() == E, "correction [E]");
    cp = correction->data_ptr();
  }
  check_hip(ks_router_topk(idx.data_ptr(), w.data_ptr(), dp, logits.data_ptr(),
                           T, E, top, softmax ? 1 : 0, renorm ? 1 : 0, cp,
                           (float)renorm_eps, (float)weight_scale,
                           current_stream()),
            "router_topk");
}

void route_tokens(at::Tensor& idx, at::Tensor& w,
                  const c10::optional<at::Tensor>& dense,
                  const c10::optional<at::Tensor>& logits_out, at::Tensor& h,
                  at::Tensor& router, bool softmax, bool renorm,
                  const c10::optional<at::Tensor>& correction,
                  double renorm_eps, double weight_scale) {
  CHECK_ROWS(h);
  CHECK_F32(router);
  CHECK_F32(w);
  CHECK_I32(idx);
  TORCH_CHECK(router.dim() == 2 && idx.dim() == 2,
              "router [E, W], idx [T, top]");
  const int T = h.size(0), W = h.size(1), E = router.size(0), top = idx.size(1);
  TORCH_CHECK(router.size(1) == W && idx.size(0) == T &&
                  w.numel() == idx.numel(),
              "route_tokens: shape mismatch");
  void *dp = nullptr, *lp = nullptr;
  if (dense.has_value()) {
    CHECK_F32(*dense);
    TORCH_CHECK(dense->numel() == (int64_t)T * E, "dense [T, E]");
    dp = dense->data_ptr();
  }
  if (logits_out.has_value()) {
    CHECK_F32(*logits_out);
    TORCH_CHECK(logits_out->numel() == (int64_t)T * E, "logits [T, E]");
    lp = logits_out->data_ptr();
  }
  const void* cp = nullptr;
  if (correction.has_value()) {
    CHECK_F32(*correction);
    TORCH_CHECK(correction->numel() == E, "correction [E]");
    cp = correction->data_ptr();
  }
  check_hip(ks_route_tokens(idx.data_ptr(), w.data_ptr(), dp, lp, h.data_ptr(),
                            h.stride(0), router.data_ptr(), T, W, E, top,
                            softmax ? 1 : 0, renorm ? 1 : 0, cp,
                            (float)renorm_eps, (float)weight_scale,
                            act_is_f32(h, "h"),
                            current_stream()),
            "route_tokens");
}

void gather_scale_rows(at::Tensor& out, at::Tensor& x, at::Tensor& rows,
                       const c10::optional<at::Tensor>& scales) {
  CHECK_ROWS(x);
  CHECK_I32(rows);
  const int f32 = act_is_f32(x, "x");
  TORCH_CHECK(out.is_contiguous() && act_is_f32(out, "out") == f32 &&
                  out.numel() == rows.numel() * x.size(1),
              "gather_scale_rows: dtype/shape mismatch");
  const void* scp = nullptr;
  if (scales.has_value()) {
    CHECK_F32(*scales);
    TORCH_CHECK(scales->numel() == rows.numel(), "scales [rows]");
    scp = scales->data_ptr();
  }
  check_hip(ks_gather_scale_rows(out.data_ptr(), x.data_ptr(), x.stride(0),
                                 rows.data_ptr(), scp,
                                 (int)rows.numel(), (int)x.size(1), f32,
                                 current_stream()),
            "gather_scale_rows");
}

void combine_rows(at::Tensor& out, at::Tensor& y, at::Tensor& index,
                  int64_t top, const c10::optional<at::Tensor>& extra,
                  const c10::optional<at::Tensor>& weights,
                  const c10::optional<at::Tensor>& scaled,
                  const c10::optional<at::Tensor>& scaled_w) {
  CHECK_F32(out);
  CHECK_I32(index);
  TORCH_CHECK(y.dim() == 2 && y.is_contiguous() && top > 0 &&
                  index.numel() % top == 0,
              "y [rows, W] contiguous, index [T * top]");
  const int f32 = act_is_f32(y, "y");
  const int tokens = index.numel() / top, width = y.size(1);
  TORCH_CHECK(out.numel() == (int64_t)tokens * width, "out [T, W]");
  const void* ep = nullptr;
  long est = 0;
  if (extra.has_value()) {
    CHECK_ROWS(*extra);
    TORCH_CHECK(act_is_f32(*extra, "extra") == f32 &&
                    extra->size(0) == tokens && extra->size(1) == width,
                "extra [T, W] in y's dtype");
    ep = extra->data_ptr();
    est = extra->stride(0);
  }
  const void *wp = nullptr, *sp = nullptr, *swp = nullptr;
  long sst = 0;
  if (weights.has_value()) {
    CHECK_F32(*weights);
    TORCH_CHECK(weights->numel() == index.numel(), "weights [T * top]");
    wp = weights->data_ptr();
  }
  if (scaled.has_value()) {
    CHECK_ROWS(*scaled);
    TORCH_CHECK(scaled_w.has_value(), "scaled rows need their weights");
    CHECK_F32(*scaled_w);
    TORCH_CHECK(act_is_f32(*scaled, "scaled") == f32 &&
                    scaled->size(0) == tokens && scaled->size(1) == width &&
                    scaled_w->numel() == tokens,
                "scaled [T, W] in y's dtype, scaled_w [T]");
    sp = scaled->data_ptr();
    sst = scaled->stride(0);
    swp = scaled_w->data_ptr();
  }
  check_hip(ks_combine_rows(out.data_ptr(), y.data_ptr(), index.data_ptr(),
                            (int)top, ep, est, tokens, width, f32, wp, sp, sst,
                            swp, current_stream()),
            "combine_rows");
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

void post_layer_norm_add(at::Tensor& residual,
                         const c10::optional<at::Tensor>& delta,
                         const c10::optional<at::Tensor>& weight, double mult,
                         double eps, const c10::optional<at::Tensor>& out,
                         const c10::optional<at::Tensor>& next_weight) {
  CHECK_F32(residual);
  TORCH_CHECK(residual.dim() == 2, "residual [T, W]");
  const int rows = residual.size(0), width = residual.size(1);
  const void *dp = nullptr, *wp = nullptr, *np = nullptr;
  void* op = nullptr;
  long dst = 0;
  int d_f32 = 1, o_f32 = 1;
  if (delta.has_value()) {
    CHECK_ROWS(*delta);
    TORCH_CHECK(weight.has_value(), "delta needs a norm weight");
    CHECK_F32(*weight);
    TORCH_CHECK(delta->size(0) == rows && delta->size(1) == width &&
                    weight->numel() == width,
                "delta / weight: shape mismatch");
    d_f32 = act_is_f32(*delta, "delta");
    dp = delta->data_ptr();
    dst = delta->stride(0);
    wp = weight->data_ptr();
  }
  if (next_weight.has_value()) {
    CHECK_F32(*next_weight);
    TORCH_CHECK(next_weight->numel() == width, "next_weight [W]");
    np = next_weight->data_ptr();
  }
  if (out.has_value()) {
    TORCH_CHECK(out->is_contiguous() && out->numel() == residual.numel(),
                "out [T, W]");
    o_f32 = act_is_f32(*out, "out");
    op = out->data_ptr();
  }
  check_hip(ks_post_layer_norm_add(residual.data_ptr(), dp, dst, d_f32, wp,
                                   (float)mult, (float)eps, op, o_f32, np, rows,
                                   width, current_stream()),
            "post_layer_norm_add");
}

void latent_norm_rope_cache(at::Tensor& cq_out, at::Tensor& proj,
                            int64_t q_rank, int64_t kv_rank, int64_t rot_dim,
                            at::Tensor& qw,
                            const c10::optional<at::Tensor>& kw,
                            at::Tensor& positions, at::Tensor& slot_mapping,
                            const c10::optional<at::Tensor>& cache, double eps,
                            const c10::optional<at::Tensor>& inv_freq) {
  CHECK_ROWS(proj);
  CHECK_F32(qw);
  CHECK_I64(positions);
  CHECK_I32(slot_mapping);
  const int f32 = act_is_f32(proj, "proj");
  const int tokens = proj.size(0);
  TORCH_CHECK(q_rank >= 1 && kv_rank >= 0 && rot_dim >= 0 &&
                  proj.size(1) >= q_rank + kv_rank + rot_dim &&
                  qw.numel() == q_rank && cq_out.is_contiguous() &&
                  act_is_f32(cq_out, "cq_out") == f32 &&
                  cq_out.numel() == (int64_t)tokens * q_rank &&
                  positions.numel() >= tokens,
              "latent_norm_rope_cache: dtype/shape mismatch");
  const void *kp = nullptr, *fp = nullptr;
  void* cp = nullptr;
  int half = 0;
  if (cache.has_value()) {
    TORCH_CHECK(kw.has_value(), "a cache needs the kv norm weight");
    CHECK_F32(*kw);
    TORCH_CHECK(cache->dim() == 4 && cache->is_contiguous() &&
                    cache->size(1) == 1 &&
                    cache->size(3) == kv_rank + rot_dim && kv_rank >= 1 &&
                    act_is_f32(*cache, "cache") == f32 &&
                    kw->numel() == kv_rank && slot_mapping.numel() >= tokens,
                "cache [blocks, 1, block, kv_rank + rot_dim] in proj's dtype");
    cp = cache->data_ptr();
    kp = kw->data_ptr();
    if (inv_freq.has_value()) {
      CHECK_F32(*inv_freq);
      half = inv_freq->numel();
      TORCH_CHECK(2 * half <= rot_dim, "more rotated pairs than the key part has");
      fp = inv_freq->data_ptr();
    }
  }
  check_hip(ks_latent_norm_rope_cache(
                cq_out.data_ptr(), proj.data_ptr(), proj.stride(0), tokens,
                (int)q_rank, (int)kv_rank, (int)rot_dim, qw.data_ptr(), kp,
                positions.data_ptr(), slot_mapping.data_ptr(), cp, (float)eps,
                fp, half, f32, current_stream()),
            "latent_norm_rope_cache");
}

void head_matmul_rope(at::Tensor& out, at::Tensor& x, at::Tensor& w,
                      int64_t heads, int64_t tail,
                      const c10::optional<at::Tensor>& positions,
                      const c10::optional<at::Tensor>& inv_freq) {
  CHECK_ROWS(x);
  TORCH_CHECK(w.dim() == 3 && w.is_contiguous() && w.size(0) == heads,
              "w [heads, n, k] contiguous");
  const int in_f32 = act_is_f32(x, "x"), out_f32 = act_is_f32(out, "out");
  const int tokens = x.size(0), N = w.size(1), K = w.size(2);
  TORCH_CHECK(act_is_f32(w, "w") == in_f32 && (out_f32 || !in_f32) &&
                  tail >= 0 && x.size(1) == heads * (K + tail) &&
                  out.is_contiguous() &&
                  out.numel() == (int64_t)tokens * heads * (N + tail),
              "head_matmul_rope: dtype/shape mismatch");
  const void *pp = nullptr, *fp = nullptr;
  int half = 0;
  if (tail > 0 && inv_freq.has_value()) {
    TORCH_CHECK(positions.has_value(), "rotation needs positions");
    CHECK_I64(*positions);
    CHECK_F32(*inv_freq);
    half = inv_freq->numel();
    TORCH_CHECK(2 * half <= tail && positions->numel() >= tokens,
                "more rotated pairs than the tail has / too few positions");
    pp = positions->data_ptr();
    fp = inv_freq->data_ptr();
  }
  check_hip(ks_head_matmul_rope(out.data_ptr(), x.data_ptr(), x.stride(0),
                                w.data_ptr(), tokens, (int)heads, K, N,
                                (int)tail, pp, fp, half, in_f32, out_f32,
                                current_stream()),
            "head_matmul_rope");
}

void glu_silu_scale(at::Tensor& out, at::Tensor& input,
                    const c10::optional<at::Tensor>& scales) {
  TORCH_CHECK(input.dim() == 2 && input.is_contiguous() && out.is_contiguous(),
              "input [rows, 2 d] contiguous");
  const int rows = input.size(0), d = input.size(1) / 2;
  const int f32 = act_is_f32(input, "input");
  TORCH_CHECK(act_is_f32(out, "out") == f32 && input.size(1) == 2 * d &&
                  out.numel() == (int64_t)rows * d,
              "glu_silu_scale: dtype/shape mismatch");
  const void* sp = nullptr;
  if (scales.has_value()) {
    CHECK_F32(*scales);
    TORCH_CHECK(scales->numel() == rows, "scales [rows]");
    sp = scales->data_ptr();
  }
  check_hip(ks_glu_silu_scale(out.data_ptr(), input.data_ptr(), sp, rows, d,
                              f32, current_stream()),
            "glu_silu_scale");
}

void relu2_scale(at::Tensor& out, at::Tensor& input,
                 const c10::optional<at::Tensor>& scales) {
  TORCH_CHECK(input.dim() == 2 && input.is_contiguous() && out.is_contiguous(),
              "input [rows, d] contiguous");
  const int rows = input.size(0), d = input.size(1);
  const int f32 = act_is_f32(input, "input");
  TORCH_CHECK(act_is_f32(out, "out") == f32 && out.numel() == input.numel(),
              "relu2_scale: dtype/shape mismatch");
  const void* sp = nullptr;
  if (scales.has_value()) {
    CHECK_F32(*scales);
    TORCH_CHECK(scales->numel() == rows, "scales [rows]");
    sp = scales->data_ptr();
  }
  check_hip(ks_relu2_scale(out.data_ptr(), input.data_ptr(), sp, rows, d, f32,
                           current_stream()),
            "relu2_scale");
}

void scale_softcap(at::Tensor& out, at::Tensor& input, double scale,
                   double cap) {
  CHECK_F32(out);
  TORCH_CHECK(input.is_contiguous() && out.numel() == input.numel(),
              "scale_softcap: shape mismatch");
  check_hip(ks_scale_softcap(out.data_ptr(), input.data_ptr(), (float)scale,
                             (float)cap, (long)input.numel(),
                             act_is_f32(input, "input"), current_stream()),
            "scale_softcap");
}

void rope_scale_heads(at::Tensor& out, at::Tensor& in, at::Tensor& positions,
                      const c10::optional<at::Tensor>& inv_freq,
                      int64_t heads_a, double scale_a, int64_t heads_b,
                      double scale_b, int64_t dim) {
  CHECK_F32(out);
  CHECK_ROWS(in);
  CHECK_I64(positions);
  const int tokens = in.size(0), width = in.size(1);
  TORCH_CHECK(heads_a >= 0 && heads_b >= 0 && dim > 0 &&
                  (heads_a + heads_b) * dim <= width &&
                  out.numel() == (int64_t)tokens * width &&
                  positions.numel() >= tokens,
              "rope_scale_heads: shape mismatch");
  const void* fp = nullptr;
  int half = 0;
  if (inv_freq.has_value()) {
    CHECK_F32(*inv_freq);
    half = inv_freq->numel();
    TORCH_CHECK(2 * half <= dim, "more rotated coordinates than the head has");
    fp = inv_freq->data_ptr();
  }
  check_hip(ks_rope_scale_heads(out.data_ptr(), in.data_ptr(), in.stride(0),
                                positions.data_ptr(), fp, half, tokens,
                                (int)heads_a, (float)scale_a, (int)heads_b,
                                (float)scale_b, (int)dim, width,
                                act_is_f32(in, "in"), current_stream()),
            "rope_scale_heads");
}

void unit_norm_heads(at::Tensor& x, int64_t heads_a, double scale_a,
                     int64_t heads_b, double scale_b, int64_t dim, double eps) {
  TORCH_CHECK(x.is_cuda() && x.scalar_type() == at::kFloat, "x must be fp32");
  CHECK_ROWS(x);
  TORCH_CHECK(heads_a >= 0 && heads_b >= 0 && dim > 0 &&
                  (heads_a + heads_b) * dim <= x.size(1),
              "unit_norm_heads: more head columns than the rows have");
  check_hip(ks_unit_norm_heads(x.data_ptr(), x.stride(0), (int)x.size(0),
                               (int)heads_a, (float)scale_a, (int)heads_b,
                               (float)scale_b, (int)dim, (float)eps,
                               current_stream()),
            "unit_norm_heads");
}

void linear_scan(at::Tensor& o, at::Tensor& q, at::Tensor& k, at::Tensor& v,
                 const c10::optional<at::Tensor>& decay,
                 const c10::optional<at::Tensor>& a_raw,
                 const c10::optional<at::Tensor>& b_raw,
                 const c10::optional<at::Tensor>& a_log,
                 const c10::optional<at::Tensor>& dt_bias, at::Tensor& state,
                 at::Tensor& positions, at::Tensor& cu_seqlens,
                 at::Tensor& slots, int64_t qk_heads) {
  CHECK_F32(o);
  CHECK_F32(state);
  CHECK_ROWS(q);
  CHECK_ROWS(k);
  CHECK_ROWS(v);
  CHECK_I64(positions);
  CHECK_I32(cu_seqlens);
  CHECK_I32(slots);
  TORCH_CHECK(q.scalar_type() == at::kFloat && k.scalar_type() == at::kFloat &&
                  v.scalar_type() == at::kFloat && q.is_cuda() && k.is_cuda() &&
                  v.is_cuda(),
              "q, k, v must be fp32 GPU tensors");
  TORCH_CHECK(state.dim() == 4, "state [slots, heads, V, K]");
  const int heads = state.size(1), V = state.size(2), K = state.size(3);
  const int tokens = q.size(0), num_seqs = slots.numel();
  TORCH_CHECK(qk_heads > 0 && heads % qk_heads == 0 &&
                  q.size(1) == qk_heads * K && k.size(1) == qk_heads * K &&
                  v.size(1) == heads * V && k.size(0) == tokens &&
                  v.size(0) == tokens &&
                  o.numel() == (int64_t)tokens * heads * V &&
                  positions.numel() >= tokens &&
                  cu_seqlens.numel() == num_seqs + 1,
              "linear_scan: shape mismatch");
  const void *dp = nullptr, *ap = nullptr, *bp = nullptr, *alp = nullptr,
             *dtp = nullptr;
  long ab_stride = 0;
  int ab_f32 = 1;
  if (decay.has_value()) {
    CHECK_F32(*decay);
    TORCH_CHECK(decay->numel() == heads, "decay [heads]");
    dp = decay->data_ptr();
  } else {
    TORCH_CHECK(a_raw.has_value() && b_raw.has_value() && a_log.has_value() &&
                    dt_bias.has_value(),
                "the delta form needs a_raw, b_raw, a_log, dt_bias");
    CHECK_ROWS(*a_raw);
    CHECK_ROWS(*b_raw);
    CHECK_F32(*a_log);
    CHECK_F32(*dt_bias);
    ab_f32 = act_is_f32(*a_raw, "a_raw");
    TORCH_CHECK(act_is_f32(*b_raw, "b_raw") == ab_f32 &&
                    a_raw->size(0) == tokens && b_raw->size(0) == tokens &&
                    a_raw->size(1) == heads && b_raw->size(1) == heads &&
                    a_raw->stride(0) == b_raw->stride(0) &&
                    a_log->numel() == heads && dt_bias->numel() == heads,
                "linear_scan: a/b shape mismatch");
    ap = a_raw->data_ptr();
    bp = b_raw->data_ptr();
    ab_stride = a_raw->stride(0);
    alp = a_log->data_ptr();
    dtp = dt_bias->data_ptr();
  }
  check_hip(ks_linear_scan(o.data_ptr(), q.data_ptr(), q.stride(0),
                           k.data_ptr(), k.stride(0), v.data_ptr(),
                           v.stride(0), dp, ap, bp, ab_stride, ab_f32, alp, dtp,
                           state.data_ptr(), positions.data_ptr(),
                           cu_seqlens.data_ptr(), slots.data_ptr(), num_seqs,
                           heads, (int)qk_heads, V, K, current_stream()),
            "linear_scan");
}

void bias_gelu_tanh(at::Tensor& out, at::Tensor& input, at::Tensor& bias) {
  TORCH_CHECK(input.dim() == 2 && input.is_contiguous() && out.is_contiguous(),
              "input [rows, d] contiguous");
  CHECK_F32(bias);
  const int rows = input.size(0), d = input.size(1);
  const int f32 = act_is_f32(input, "input");
  TORCH_CHECK(act_is_f32(out, "out") == f32 && out.numel() == input.numel() &&
                  bias.numel() == d,
              "bias_gelu_tanh: dtype/shape mismatch");
  check_hip(ks_bias_gelu_tanh(out.data_ptr(), input.data_ptr(), bias.data_ptr(),
                              rows, d, f32, current_stream()),
            "bias_gelu_tanh");
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
  m.def("qk_headnorm_rope_cache", &qk_headnorm_rope_cache,
        "per-head q/k RMS norm + rotary, optional value norm/rotation, KV scatter");
  m.def("post_norm_add_rms_norm", &post_norm_add_rms_norm,
        "fp32 residual += layer_scale * post-norm(delta) (+ rows, + row), then RMS norm");
  m.def("router_topk", &router_topk, "sigmoid/softmax scores and top-k experts");
  m.def("route_tokens", &route_tokens,
        "fp32 router logits + sigmoid/softmax scores + top-k experts, fused");
  m.def("gather_scale_rows", &gather_scale_rows, "out[r] = x[rows[r]] * scales[r]");
  m.def("combine_rows", &combine_rows, "fp32 sum of indexed rows per token");
  m.def("post_layer_norm_add", &post_layer_norm_add,
        "fp32 residual += mult * LayerNorm(delta) * w, then cast or final layer norm");
  m.def("latent_norm_rope_cache", &latent_norm_rope_cache,
        "RMS norm of query / kv latents, pair rotation of the key part, page scatter");
  m.def("head_matmul_rope", &head_matmul_rope,
        "per-head matrix product with an optional pair-rotated tail");
  m.def("glu_silu_scale", &glu_silu_scale, "silu(gate) * up * row scale");
  m.def("bias_gelu_tanh", &bias_gelu_tanh, "gelu (tanh form) of x + bias");
  m.def("relu2_scale", &relu2_scale, "max(x, 0)^2 * row scale");
  m.def("scale_softcap", &scale_softcap, "cap * tanh(x * scale / cap), fp32");
  m.def("rope_scale_heads", &rope_scale_heads,
        "rotary positions on projection heads, times a constant, fp32 out");
  m.def("unit_norm_heads", &unit_norm_heads,
        "per-head unit vectors times a constant, in place");
  m.def("linear_scan", &linear_scan,
        "decay / gated-delta linear-attention recurrence, per-slot fp32 state");
  def_sampling(m);
}
