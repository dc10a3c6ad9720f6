// Torch operator registration of the sequence-mixer kernels (namespace `atta_mix`).  Every op
// checks shapes, dtypes and strides on the host against what its kernel and grid assume, then
// launches on the current stream: no allocation, no synchronisation, safe under graph capture.
#include <torch/library.h>
#include <ATen/ATen.h>
#include <c10/hip/HIPStream.h>
#include <c10/core/DeviceGuard.h>

#include "mixers.h"

namespace {

hipStream_t cur_stream() { return c10::hip::getCurrentHIPStream().stream(); }

int code(const at::Tensor& t) {
  if (t.scalar_type() == at::kBFloat16) return 0;
  if (t.scalar_type() == at::kFloat) return 2;
  TORCH_CHECK(false, "atta_mix: expected a bf16 or fp32 tensor, got ", t.scalar_type());
}

void rc_ok(int rc, const char* what) {
  TORCH_CHECK(rc == 0, "atta_mix::", what, " launch failed (rc=", rc, ")");
}

void i32(const at::Tensor& t, const char* name) {
  TORCH_CHECK(t.is_cuda() && t.scalar_type() == at::kInt && t.is_contiguous(), "atta_mix: ", name,
              " must be a contiguous int32 GPU tensor");
}

void f32c(const at::Tensor& t, const char* name) {
  TORCH_CHECK(t.is_cuda() && t.scalar_type() == at::kFloat && t.is_contiguous(), "atta_mix: ",
              name, " must be a contiguous fp32 GPU tensor");
}

// activation tensor [rows, cols] with unit column stride, dtype of `like`
void rows2d(const at::Tensor& t, const at::Tensor& like, const char* name) {
  TORCH_CHECK(t.is_cuda() && t.dim() == 2 && t.stride(1) == 1 && t.scalar_type() == like.scalar_type(),
              "atta_mix: ", name, " must be a 2-D GPU tensor with unit column stride");
}

void meta(const at::Tensor& positions, const at::Tensor& seq_qstart, const at::Tensor& seq_slot,
          int64_t T) {
  i32(positions, "positions");
  i32(seq_qstart, "seq_qstart");
  i32(seq_slot, "seq_slot");
  TORCH_CHECK(positions.numel() >= T && seq_qstart.numel() == seq_slot.numel() + 1,
              "atta_mix: metadata sizes");
}

void embed_pair(at::Tensor out, const at::Tensor& table, const at::Tensor& pair_table,
                const at::Tensor& ids, const at::Tensor& positions, const at::Tensor& seq_qstart,
                const at::Tensor& seq_slot, at::Tensor prev_token, int64_t mul_prev,
                int64_t mul_cur, int64_t buckets) {
  const int64_t T = ids.numel(), W = table.size(1);
  i32(ids, "ids");
  meta(positions, seq_qstart, seq_slot, T);
  i32(prev_token, "prev_token");
  f32c(out, "out");
  TORCH_CHECK(table.is_cuda() && table.is_contiguous() && pair_table.is_contiguous() &&
                  pair_table.scalar_type() == table.scalar_type() && pair_table.size(1) == W &&
                  pair_table.size(0) == buckets + 1 && out.size(0) == T && out.size(1) == W &&
                  buckets > 0,
              "embed_pair: table shapes");
  const at::DeviceGuard g(table.device());
  rc_ok(mixk_embed_pair(out.data_ptr<float>(), table.data_ptr(), pair_table.data_ptr(),
                        ids.data_ptr<int>(), positions.data_ptr<int>(), seq_qstart.data_ptr<int>(),
                        seq_slot.data_ptr<int>(), prev_token.data_ptr<int>(), T, seq_slot.numel(),
                        W, mul_prev, mul_cur, buckets, code(table), cur_stream()),
        "embed_pair");
}

void rms_norm_f32(at::Tensor out, const at::Tensor& x, const at::Tensor& w, double eps,
                  bool one_plus) {
  f32c(x, "x");
  TORCH_CHECK(x.dim() == 2 && out.is_cuda() && out.is_contiguous() && out.sizes() == x.sizes() &&
                  w.is_contiguous() && w.numel() == x.size(1) &&
                  w.scalar_type() == out.scalar_type(),
              "rms_norm_f32: shapes");
  const at::DeviceGuard g(x.device());
  rc_ok(mixk_rms_norm_f32(out.data_ptr(), x.data_ptr<float>(), w.data_ptr(), x.size(0), x.size(1),
                          static_cast<float>(eps), one_plus, code(out), cur_stream()),
        "rms_norm_f32");
}

void relu_sq(at::Tensor out, const at::Tensor& x) {
  rows2d(x, out, "x");
  TORCH_CHECK(out.is_contiguous() && out.sizes() == x.sizes(), "relu_sq: out");
  const at::DeviceGuard g(x.device());
  rc_ok(mixk_relu_sq(out.data_ptr(), x.data_ptr(), x.size(0), x.size(1), x.stride(0), code(x),
                     cur_stream()),
        "relu_sq");
}

void residual_add(at::Tensor x, const at::Tensor& a, double sa, const c10::optional<at::Tensor>& b,
                  double sb, const c10::optional<at::Tensor>& c) {
  f32c(x, "x");
  auto same = [&](const at::Tensor& t) {
    TORCH_CHECK(t.is_cuda() && t.is_contiguous() && t.numel() == x.numel() &&
                    t.scalar_type() == a.scalar_type(),
                "residual_add: branch shapes");
  };
  same(a);
  if (b) same(*b);
  if (c) same(*c);
  const at::DeviceGuard g(x.device());
  rc_ok(mixk_residual_add(x.data_ptr<float>(), a.data_ptr(), static_cast<float>(sa),
                          b ? b->data_ptr() : nullptr, static_cast<float>(sb),
                          c ? c->data_ptr() : nullptr, x.numel(), code(a), cur_stream()),
        "residual_add");
}

void add_norm(at::Tensor h, at::Tensor x, const at::Tensor& a, double sa,
              const c10::optional<at::Tensor>& b, double sb, const c10::optional<at::Tensor>& c,
              const at::Tensor& w, double eps, bool one_plus) {
  f32c(x, "x");
  TORCH_CHECK(x.dim() == 2 && h.is_cuda() && h.is_contiguous() && h.sizes() == x.sizes() &&
                  w.is_contiguous() && w.numel() == x.size(1) &&
                  w.scalar_type() == h.scalar_type() && a.scalar_type() == h.scalar_type(),
              "add_norm: shapes");
  auto same = [&](const at::Tensor& t) {
    TORCH_CHECK(t.is_cuda() && t.is_contiguous() && t.numel() == x.numel() &&
                    t.scalar_type() == a.scalar_type(),
                "add_norm: branch shapes");
  };
  same(a);
  if (b) same(*b);
  if (c) same(*c);
  const at::DeviceGuard g(x.device());
  rc_ok(mixk_add_norm(h.data_ptr(), x.data_ptr<float>(), a.data_ptr(), static_cast<float>(sa),
                      b ? b->data_ptr() : nullptr, static_cast<float>(sb),
                      c ? c->data_ptr() : nullptr, w.data_ptr(), x.size(0), x.size(1),
                      static_cast<float>(eps), one_plus, code(h), cur_stream()),
        "add_norm");
}

void gated_rms_norm(at::Tensor out, const at::Tensor& o, const at::Tensor& gate,
                    const at::Tensor& w, double eps, int64_t act) {
  f32c(o, "o");
  TORCH_CHECK(o.dim() == 3, "gated_rms_norm: o [T, H, dv]");
  const int64_t T = o.size(0), H = o.size(1), dv = o.size(2);
  rows2d(gate, out, "gate");
  TORCH_CHECK(gate.size(0) == T && gate.size(1) == H * dv && out.is_contiguous() &&
                  out.numel() == o.numel() && w.is_contiguous() && w.numel() == dv &&
                  w.scalar_type() == out.scalar_type(),
              "gated_rms_norm: shapes");
  const at::DeviceGuard g(o.device());
  rc_ok(mixk_gated_rms_norm(out.data_ptr(), o.data_ptr<float>(), gate.data_ptr(), gate.stride(0),
                            w.data_ptr(), T, H, dv, static_cast<float>(eps), act, code(out),
                            cur_stream()),
        "gated_rms_norm");
}

void qk_norm_rope_cache(at::Tensor q_out, const at::Tensor& qx, const at::Tensor& kx,
                        const at::Tensor& vx, const c10::optional<at::Tensor>& q_norm,
                        const c10::optional<at::Tensor>& k_norm, double eps,
                        const at::Tensor& positions, const at::Tensor& slot_mapping,
                        const at::Tensor& cos_sin, at::Tensor k_cache, at::Tensor v_cache,
                        bool rotate_half, bool norm_last,
                        const c10::optional<at::Tensor>& row_inv) {
  TORCH_CHECK(q_out.dim() == 3 && q_out.is_contiguous() && k_cache.dim() == 4 &&
                  v_cache.dim() == 4 && k_cache.is_contiguous() && v_cache.is_contiguous(),
              "qk_norm_rope_cache: q_out [T, H, d], caches [nb, G, BS, d]");
  const int64_t T = q_out.size(0), H = q_out.size(1), dim = q_out.size(2);
  const int64_t G = k_cache.size(1), BS = k_cache.size(2), vdim = v_cache.size(2);
  rows2d(qx, q_out, "q");
  rows2d(kx, q_out, "k");
  rows2d(vx, q_out, "v");
  i32(positions, "positions");
  i32(slot_mapping, "slot_mapping");
  f32c(cos_sin, "cos_sin");
  TORCH_CHECK(cos_sin.dim() == 2 && cos_sin.size(0) >= T && cos_sin.size(1) % 2 == 0,
              "qk_norm_rope_cache: cos_sin [rows, 2 n_freq]");
  const int64_t n_freq = cos_sin.size(1) / 2;
  TORCH_CHECK(qx.size(0) == T && kx.size(0) == T && vx.size(0) == T && qx.size(1) == H * dim &&
                  kx.size(1) == G * dim && vx.size(1) == G * vdim && k_cache.size(3) == dim &&
                  v_cache.size(1) == G && v_cache.size(3) == BS &&
                  v_cache.size(0) == k_cache.size(0) && positions.numel() >= T &&
                  slot_mapping.numel() >= T && 2 * n_freq <= dim &&
                  k_cache.scalar_type() == q_out.scalar_type() &&
                  v_cache.scalar_type() == q_out.scalar_type(),
              "qk_norm_rope_cache: shapes");
  // row_inv [T, 2]: the inverse RMS of the whole q / k projection of every row; the weights then
  // cover the projection, [H * dim] and [G * dim]
  if (row_inv) {
    f32c(*row_inv, "row_inv");
    TORCH_CHECK(row_inv->numel() == 2 * T && !norm_last, "qk_norm_rope_cache: row_inv [T, 2]");
  }
  int64_t heads_of = H;
  for (const auto* w : {&q_norm, &k_norm}) {
    if (w->has_value())
      TORCH_CHECK((*w)->is_cuda() && (*w)->numel() == (row_inv ? heads_of * dim : dim) &&
                      (*w)->is_contiguous() && (*w)->scalar_type() == q_out.scalar_type(),
                  "qk_norm_rope_cache: norm weights [dim] (or [heads * dim] with row_inv)");
    heads_of = G;
  }
  const at::DeviceGuard g(qx.device());
  rc_ok(mixk_qk_norm_rope_cache(q_out.data_ptr(), qx.data_ptr(), qx.stride(0), kx.data_ptr(),
                                kx.stride(0), vx.data_ptr(), vx.stride(0),
                                q_norm ? q_norm->data_ptr() : nullptr,
                                k_norm ? k_norm->data_ptr() : nullptr, static_cast<float>(eps),
                                positions.data_ptr<int>(), slot_mapping.data_ptr<int>(),
                                cos_sin.data_ptr<float>(), n_freq, k_cache.data_ptr(),
                                v_cache.data_ptr(), T, H, G, dim, vdim, BS, rotate_half, norm_last,
                                row_inv ? row_inv->data_ptr<float>() : nullptr, code(q_out),
                                cur_stream()),
        "qk_norm_rope_cache");
}

void rotary_table(at::Tensor out, const at::Tensor& positions, const at::Tensor& inv_freq) {
  i32(positions, "positions");
  f32c(inv_freq, "inv_freq");
  f32c(out, "out");
  TORCH_CHECK(out.dim() == 2 && out.size(1) == 2 * inv_freq.numel() &&
                  positions.numel() >= out.size(0),
              "rotary_table: out [rows, 2 n_freq]");
  const at::DeviceGuard g(out.device());
  rc_ok(mixk_rotary_table(out.data_ptr<float>(), positions.data_ptr<int>(),
                          inv_freq.data_ptr<float>(), out.size(0), inv_freq.numel(), cur_stream()),
        "rotary_table");
}

void sink_attention(at::Tensor out, const at::Tensor& q, const at::Tensor& k_cache,
                    const at::Tensor& v_cache, const at::Tensor& block_tables,
                    const at::Tensor& seq_kvlen, const at::Tensor& seq_qstart,
                    const at::Tensor& tile_seq, const at::Tensor& tile_qoff, double scale,
                    bool sink, int64_t num_decode, int64_t max_decode_kv,
                    const c10::optional<at::Tensor>& part, bool use_mfma,
                    const c10::optional<at::Tensor>& sink_val, int64_t window) {
  TORCH_CHECK(q.is_cuda() && q.dim() == 3 && q.is_contiguous() && out.dim() == 3 &&
                  out.is_contiguous() && k_cache.dim() == 4 && v_cache.dim() == 4 &&
                  k_cache.is_contiguous() && v_cache.is_contiguous(),
              "sink_attention: q [T, H, d], out [T, H, dv], K [nb, G, BS, d], V [nb, G, dv, BS]");
  const int64_t H = q.size(1), dim = q.size(2), G = k_cache.size(1), BS = k_cache.size(2);
  const int64_t vdim = v_cache.size(2), S = seq_kvlen.numel();
  i32(block_tables, "block_tables");
  i32(seq_kvlen, "seq_kvlen");
  i32(seq_qstart, "seq_qstart");
  i32(tile_seq, "tile_seq");
  i32(tile_qoff, "tile_qoff");
  TORCH_CHECK(block_tables.dim() == 2 && block_tables.size(0) >= S &&
                  seq_qstart.numel() == S + 1 && tile_seq.numel() == tile_qoff.numel() &&
                  out.size(0) == q.size(0) && out.size(1) == H && out.size(2) == vdim &&
                  k_cache.size(3) == dim && v_cache.size(1) == G && v_cache.size(3) == BS &&
                  v_cache.size(0) == k_cache.size(0) && H % G == 0 &&
                  out.scalar_type() == q.scalar_type() &&
                  k_cache.scalar_type() == q.scalar_type() &&
                  v_cache.scalar_type() == q.scalar_type() && num_decode >= 0 && num_decode <= S,
              "sink_attention: shapes");
  float* part_ptr = nullptr;
  int64_t max_parts = 0;
  if (num_decode > 0) {
    TORCH_CHECK(part.has_value(), "sink_attention: decode rows need the partials workspace");
    f32c(*part, "part");
    TORCH_CHECK(part->dim() == 4 && part->size(0) >= num_decode && part->size(1) == H &&
                    part->size(3) == vdim + 2 && max_decode_kv >= 1 && window >= 0 &&
                    (part->size(2) * 128 >= max_decode_kv ||
                     (window > 0 && part->size(2) >= (window + 127) / 128 + 1)),
                "sink_attention: partials [num_decode, H, parts, vdim + 2]");
    part_ptr = part->data_ptr<float>();
    max_parts = part->size(2);
  }
  if (use_mfma)
    TORCH_CHECK(q.scalar_type() == at::kBFloat16 && dim % 16 == 0 && vdim % 32 == 0 &&
                    dim <= 256 && vdim <= 256 && BS >= 8 && (BS & (BS - 1)) == 0,
                "sink_attention: matrix-core kernel needs bf16, dim % 16, vdim % 32, <= 256, "
                "pages of a power of two >= 8 tokens");
  const float* sink_ptr = nullptr;
  if (sink_val) {
    f32c(*sink_val, "sink_val");
    TORCH_CHECK(sink && sink_val->numel() == H, "sink_attention: sink_val [H] needs sink");
    sink_ptr = sink_val->data_ptr<float>();
  }
  const at::DeviceGuard g(q.device());
  rc_ok(mixk_sink_attention(out.data_ptr(), q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(),
                            block_tables.data_ptr<int>(), block_tables.size(1),
                            seq_kvlen.data_ptr<int>(), seq_qstart.data_ptr<int>(),
                            tile_seq.data_ptr<int>(), tile_qoff.data_ptr<int>(), tile_seq.numel(),
                            num_decode, max_decode_kv, part_ptr, max_parts, H, G, dim, vdim, BS,
                            static_cast<float>(scale), sink, sink_ptr, static_cast<int>(window),
                            use_mfma, code(q), cur_stream()),
        "sink_attention");
}

void short_conv_silu(at::Tensor out, const at::Tensor& x, const at::Tensor& w,
                     at::Tensor conv_state, const at::Tensor& positions,
                     const at::Tensor& seq_qstart, const at::Tensor& seq_slot,
                     const c10::optional<at::Tensor>& bias) {
  rows2d(x, out, "x");
  const int64_t T = x.size(0), C = x.size(1);
  meta(positions, seq_qstart, seq_slot, T);
  TORCH_CHECK(w.dim() == 2 && w.is_contiguous() && w.size(0) == C && out.is_contiguous() &&
                  out.size(0) == T && out.size(1) == C && w.scalar_type() == x.scalar_type(),
              "short_conv_silu: shapes");
  const int64_t taps = w.size(1);
  if (taps > 1)
    TORCH_CHECK(conv_state.is_cuda() && conv_state.is_contiguous() && conv_state.dim() == 3 &&
                    conv_state.size(1) == taps - 1 && conv_state.size(2) == C &&
                    conv_state.scalar_type() == x.scalar_type(),
                "short_conv_silu: conv_state [slots, taps - 1, C]");
  if (bias)
    TORCH_CHECK(bias->is_cuda() && bias->is_contiguous() && bias->numel() == C &&
                    bias->scalar_type() == x.scalar_type(),
                "short_conv_silu: bias [C]");
  const at::DeviceGuard g(x.device());
  rc_ok(mixk_short_conv_silu(out.data_ptr(), x.data_ptr(), x.stride(0), w.data_ptr(),
                             bias ? bias->data_ptr() : nullptr, conv_state.data_ptr(), positions.data_ptr<int>(),
                             seq_qstart.data_ptr<int>(), seq_slot.data_ptr<int>(), T,
                             seq_slot.numel(), C, taps, code(x), cur_stream()),
        "short_conv_silu");
}

void gated_delta_rule(at::Tensor out, const at::Tensor& qkv, const at::Tensor& beta,
                      const at::Tensor& decay, const at::Tensor& a_log, const at::Tensor& dt_bias,
                      at::Tensor state, const at::Tensor& positions, const at::Tensor& seq_qstart,
                      const at::Tensor& seq_slot, int64_t H, int64_t G, int64_t dim,
                      int64_t vdim) {
  TORCH_CHECK(qkv.is_cuda() && qkv.dim() == 2 && qkv.is_contiguous() &&
                  qkv.size(1) == 2 * G * dim + H * vdim,
              "gated_delta_rule: qkv [T, 2 G d + H dv]");
  const int64_t T = qkv.size(0);
  rows2d(beta, qkv, "beta");
  rows2d(decay, qkv, "decay");
  meta(positions, seq_qstart, seq_slot, T);
  f32c(out, "out");
  f32c(a_log, "a_log");
  f32c(dt_bias, "dt_bias");
  f32c(state, "state");
  const bool per_channel = decay.size(1) == H * dim && dt_bias.numel() == H * dim;
  TORCH_CHECK(beta.size(0) == T && beta.size(1) == H && decay.size(0) == T &&
                  (per_channel || (decay.size(1) == H && dt_bias.numel() == H)) &&
                  a_log.numel() == H && out.numel() == T * H * vdim && state.dim() == 4 &&
                  state.size(1) == H && state.size(2) == dim && state.size(3) == vdim &&
                  H % G == 0 && dim <= 256,
              "gated_delta_rule: shapes");
  const at::DeviceGuard g(qkv.device());
  rc_ok(mixk_gated_delta_rule(out.data_ptr<float>(), qkv.data_ptr(), beta.data_ptr(),
                              beta.stride(0), decay.data_ptr(), decay.stride(0), per_channel,
                              a_log.data_ptr<float>(), dt_bias.data_ptr<float>(),
                              state.data_ptr<float>(), positions.data_ptr<int>(),
                              seq_qstart.data_ptr<int>(), seq_slot.data_ptr<int>(),
                              seq_slot.numel(), H, G, dim, vdim, code(qkv), cur_stream()),
        "gated_delta_rule");
}


void embed_scale(at::Tensor out, const at::Tensor& table, const at::Tensor& ids, double scale) {
  i32(ids, "ids");
  f32c(out, "out");
  // out [T, W], or [T, copies, W]: the row written `copies` times
  TORCH_CHECK(table.is_cuda() && table.dim() == 2 && table.is_contiguous() &&
                  (out.dim() == 2 || out.dim() == 3) && out.size(0) == ids.numel() &&
                  out.size(out.dim() - 1) == table.size(1),
              "embed_scale: shapes");
  const at::DeviceGuard g(table.device());
  rc_ok(mixk_embed_scale(out.data_ptr<float>(), table.data_ptr(), ids.data_ptr<int>(),
                         ids.numel(), table.size(1), table.size(0), static_cast<float>(scale),
                         out.dim() == 3 ? out.size(1) : 1, code(table), cur_stream()),
        "embed_scale");
}

void rms_norm_rows(at::Tensor out, const at::Tensor& x, const at::Tensor& w, double eps) {
  rows2d(x, out, "x");
  TORCH_CHECK(out.is_contiguous() && out.sizes() == x.sizes() && w.is_cuda() &&
                  w.is_contiguous() && w.numel() == x.size(1) &&
                  w.scalar_type() == x.scalar_type(),
              "rms_norm_rows: shapes");
  const at::DeviceGuard g(x.device());
  rc_ok(mixk_rms_norm_rows(out.data_ptr(), x.data_ptr(), x.stride(0), w.data_ptr(), x.size(0),
                           x.size(1), static_cast<float>(eps), code(x), cur_stream()),
        "rms_norm_rows");
}

void xielu_bias(at::Tensor out, const at::Tensor& x, const c10::optional<at::Tensor>& bias,
                double ap, double aq) {
  rows2d(x, out, "x");
  TORCH_CHECK(out.is_contiguous() && out.sizes() == x.sizes(), "xielu_bias: out");
  if (bias)
    TORCH_CHECK(bias->is_cuda() && bias->is_contiguous() && bias->numel() == x.size(1) &&
                    bias->scalar_type() == x.scalar_type(),
                "xielu_bias: bias [N]");
  const at::DeviceGuard g(x.device());
  rc_ok(mixk_xielu_bias(out.data_ptr(), x.data_ptr(), x.stride(0),
                        bias ? bias->data_ptr() : nullptr, x.size(0), x.size(1),
                        static_cast<float>(ap), static_cast<float>(aq), code(x), cur_stream()),
        "xielu_bias");
}

void group_rms_norm(at::Tensor out, const at::Tensor& y, const c10::optional<at::Tensor>& gate,
                    const at::Tensor& w, int64_t n_groups, double eps) {
  f32c(y, "y");
  TORCH_CHECK(y.dim() == 2 && n_groups > 0 && y.size(1) % n_groups == 0, "group_rms_norm: y [T, n gs]");
  const int64_t T = y.size(0), N = y.size(1), gs = N / n_groups;
  TORCH_CHECK(out.is_cuda() && out.is_contiguous() && out.dim() == 2 && out.size(0) == T &&
                  out.size(1) == N && w.is_cuda() && w.is_contiguous() &&
                  (w.numel() == gs || w.numel() == N) && w.scalar_type() == out.scalar_type(),
              "group_rms_norm: shapes");
  int64_t gstride = 0;
  if (gate) {
    rows2d(*gate, out, "gate");
    TORCH_CHECK(gate->size(0) == T && gate->size(1) == N, "group_rms_norm: gate [T, n gs]");
    gstride = gate->stride(0);
  }
  const at::DeviceGuard g(y.device());
  rc_ok(mixk_group_rms_norm(out.data_ptr(), y.data_ptr<float>(),
                            gate ? gate->data_ptr() : nullptr, gstride, w.data_ptr(), T, n_groups,
                            gs, static_cast<float>(eps), w.numel() == N && n_groups > 1,
                            code(out), cur_stream()),
        "group_rms_norm");
}

void head_gate(at::Tensor out, const at::Tensor& o, const at::Tensor& gate) {
  TORCH_CHECK(o.is_cuda() && o.dim() == 3 && o.is_contiguous(), "head_gate: o [H, T, dv]");
  const int64_t H = o.size(0), T = o.size(1), dv = o.size(2);
  rows2d(gate, o, "gate");
  TORCH_CHECK(gate.size(0) == T && gate.size(1) == H && out.is_contiguous() &&
                  out.numel() == o.numel() && out.scalar_type() == o.scalar_type(),
              "head_gate: shapes");
  const at::DeviceGuard g(o.device());
  rc_ok(mixk_head_gate(out.data_ptr(), o.data_ptr(), gate.data_ptr(), gate.stride(0), T, H, dv,
                       code(o), cur_stream()),
        "head_gate");
}

void latent_rope_cache(at::Tensor q_out, const at::Tensor& q_lat, const at::Tensor& qx,
                       const c10::optional<at::Tensor>& kvx, const c10::optional<at::Tensor>& c_norm,
                       double eps, const at::Tensor& slot_mapping, const at::Tensor& cos_sin,
                       at::Tensor k_cache, at::Tensor v_cache, at::Tensor c_out) {
  TORCH_CHECK(q_out.is_cuda() && q_out.dim() == 3 && q_out.is_contiguous() && q_lat.dim() == 3 &&
                  q_lat.is_contiguous() && qx.dim() == 3 && qx.is_contiguous() &&
                  k_cache.dim() == 4 && v_cache.dim() == 4 && k_cache.is_contiguous() &&
                  v_cache.is_contiguous(),
              "latent_rope_cache: q_out [T, H, rank + rot], q_lat [H, T, rank], qx [T, H, qdim + rot]");
  const int64_t T = q_out.size(0), H = q_out.size(1), kd = q_out.size(2), rank = q_lat.size(2);
  const int64_t rot = kd - rank, qdim = qx.size(2) - rot, BS = k_cache.size(2);
  i32(slot_mapping, "slot_mapping");
  f32c(cos_sin, "cos_sin");
  TORCH_CHECK(cos_sin.dim() == 2 && cos_sin.size(0) >= T && cos_sin.size(1) % 2 == 0,
              "latent_rope_cache: cos_sin [rows, 2 n_freq]");
  const int64_t n_freq = cos_sin.size(1) / 2;
  TORCH_CHECK(rot >= 0 && qdim >= 0 && 2 * n_freq <= rot && q_lat.size(0) == H &&
                  q_lat.size(1) == T && qx.size(0) == T && qx.size(1) == H &&
                  k_cache.size(1) == 1 && k_cache.size(3) == kd && v_cache.size(1) == 1 &&
                  v_cache.size(2) == rank && v_cache.size(3) == BS &&
                  v_cache.size(0) == k_cache.size(0) && slot_mapping.numel() >= T &&
                  q_lat.scalar_type() == q_out.scalar_type() &&
                  qx.scalar_type() == q_out.scalar_type() &&
                  k_cache.scalar_type() == q_out.scalar_type() &&
                  v_cache.scalar_type() == q_out.scalar_type(),
              "latent_rope_cache: shapes");
  const void* kv_ptr = nullptr;
  const void* norm_ptr = nullptr;
  int64_t kv_stride = 0;
  if (kvx) {
    rows2d(*kvx, q_out, "kvx");
    TORCH_CHECK(c_norm.has_value() && c_norm->is_cuda() && c_norm->is_contiguous() &&
                    c_norm->numel() == rank && c_norm->scalar_type() == q_out.scalar_type() &&
                    kvx->size(0) == T && kvx->size(1) == kd && c_out.is_cuda() &&
                    c_out.is_contiguous() && c_out.numel() >= T * rank &&
                    c_out.scalar_type() == q_out.scalar_type(),
                "latent_rope_cache: kvx [T, rank + rot], c_norm [rank], c_out [T, rank]");
    kv_ptr = kvx->data_ptr();
    norm_ptr = c_norm->data_ptr();
    kv_stride = kvx->stride(0);
  }
  const at::DeviceGuard g(q_out.device());
  rc_ok(mixk_latent_rope_cache(q_out.data_ptr(), q_lat.data_ptr(), qx.data_ptr(), kv_ptr,
                               kv_stride, norm_ptr, static_cast<float>(eps),
                               slot_mapping.data_ptr<int>(), cos_sin.data_ptr<float>(), n_freq,
                               k_cache.data_ptr(), v_cache.data_ptr(), c_out.data_ptr(), T, H,
                               qdim, rank, rot, BS, code(q_out), cur_stream()),
        "latent_rope_cache");
}

// mode 0 (forget gate): q = q_raw [T, H dk], k = f [T, H dk], p0 = f_bias [H dk], p1 = lower [H dk].
// mode 1 (state space): q = C [T, G dk], k = B [T, G dk], dt [T, H], p0 = dt_bias [H],
// p1 = A_log [H], p2 = D [H].
void gated_linear_scan(at::Tensor out, at::Tensor state, const at::Tensor& q, const at::Tensor& k,
                       const at::Tensor& v, const c10::optional<at::Tensor>& dt,
                       const at::Tensor& p0, const at::Tensor& p1,
                       const c10::optional<at::Tensor>& p2, const at::Tensor& positions,
                       const at::Tensor& seq_qstart, const at::Tensor& seq_slot, int64_t H,
                       int64_t G, int64_t dk, int64_t dv, int64_t mode) {
  TORCH_CHECK(v.is_cuda() && v.dim() == 2 && v.stride(1) == 1, "gated_linear_scan: v [T, H dv]");
  const int64_t T = v.size(0);
  rows2d(q, v, "q");
  rows2d(k, v, "k");
  meta(positions, seq_qstart, seq_slot, T);
  f32c(out, "out");
  f32c(state, "state");
  f32c(p0, "p0");
  f32c(p1, "p1");
  TORCH_CHECK(mode == 0 || mode == 1, "gated_linear_scan: mode");
  const int64_t qk_cols = (mode == 0 ? H : G) * dk;
  TORCH_CHECK(H > 0 && G > 0 && dk > 0 && dk <= 256 && dv > 0 && v.size(1) == H * dv &&
                  q.size(0) == T && k.size(0) == T && q.size(1) == qk_cols &&
                  k.size(1) == qk_cols && out.numel() == T * H * dv && state.dim() == 4 &&
                  state.size(1) == H && state.size(2) == dk && state.size(3) == dv,
              "gated_linear_scan: shapes");
  const void* dt_ptr = nullptr;
  const float* p2_ptr = nullptr;
  int64_t dt_stride = 0;
  if (mode == 0) {
    TORCH_CHECK(p0.numel() == H * dk && p1.numel() == H * dk, "gated_linear_scan: f_bias, lower [H dk]");
  } else {
    TORCH_CHECK(dt.has_value() && p2.has_value() && H % G == 0 && p0.numel() == H &&
                    p1.numel() == H && p2->numel() == H,
                "gated_linear_scan: dt [T, H], dt_bias / A_log / D [H]");
    rows2d(*dt, v, "dt");
    f32c(*p2, "p2");
    TORCH_CHECK(dt->size(0) == T && dt->size(1) == H, "gated_linear_scan: dt [T, H]");
    dt_ptr = dt->data_ptr();
    dt_stride = dt->stride(0);
    p2_ptr = p2->data_ptr<float>();
  }
  const at::DeviceGuard g(v.device());
  rc_ok(mixk_gated_linear_scan(out.data_ptr<float>(), state.data_ptr<float>(), q.data_ptr(),
                               q.stride(0), k.data_ptr(), k.stride(0), v.data_ptr(), v.stride(0),
                               dt_ptr, dt_stride, p0.data_ptr<float>(), p1.data_ptr<float>(),
                               p2_ptr, positions.data_ptr<int>(), seq_qstart.data_ptr<int>(),
                               seq_slot.data_ptr<int>(), seq_slot.numel(), H, G, dk, dv, mode,
                               code(v), cur_stream()),
        "gated_linear_scan");
}

void hyper_update_norm(const c10::optional<at::Tensor>& out, at::Tensor xs,
                       const c10::optional<at::Tensor>& y, const c10::optional<at::Tensor>& mix,
                       const c10::optional<at::Tensor>& w_out,
                       const c10::optional<at::Tensor>& w_in, const c10::optional<at::Tensor>& w,
                       double eps) {
  f32c(xs, "xs");
  TORCH_CHECK(xs.dim() == 3 && xs.size(1) >= 1 && xs.size(1) <= 8, "hyper_update_norm: xs [T, s, W]");
  const int64_t T = xs.size(0), ns = xs.size(1), W = xs.size(2);
  TORCH_CHECK(y.has_value() || w.has_value(), "hyper_update_norm: nothing to do");
  int dt = -1;
  if (y) {
    TORCH_CHECK(y->is_cuda() && y->is_contiguous() && y->dim() == 2 && y->size(0) == T &&
                    y->size(1) == W && mix.has_value() && w_out.has_value(),
                "hyper_update_norm: y [T, W] with mix and w_out");
    f32c(*mix, "mix");
    f32c(*w_out, "w_out");
    TORCH_CHECK(mix->numel() == ns * ns && w_out->numel() == ns, "hyper_update_norm: mix [s, s]");
    dt = code(*y);
  }
  if (w) {
    TORCH_CHECK(out.has_value() && w_in.has_value(), "hyper_update_norm: norm needs out and w_in");
    f32c(*w_in, "w_in");
    TORCH_CHECK(w->is_cuda() && w->is_contiguous() && w->numel() == W && w_in->numel() == ns &&
                    out->is_cuda() && out->is_contiguous() && out->dim() == 2 &&
                    out->size(0) == T && out->size(1) == W && (dt < 0 || dt == code(*w)) &&
                    (out->scalar_type() == at::kFloat || out->scalar_type() == w->scalar_type()),
                "hyper_update_norm: out [T, W] fp32 or of the weight's dtype");
    dt = code(*w);
  }
  const at::DeviceGuard g(xs.device());
  rc_ok(mixk_hyper_update_norm(w ? out->data_ptr() : nullptr,
                               w && out->scalar_type() == at::kFloat, xs.data_ptr<float>(),
                               y ? y->data_ptr() : nullptr, y ? mix->data_ptr<float>() : nullptr,
                               y ? w_out->data_ptr<float>() : nullptr,
                               w ? w_in->data_ptr<float>() : nullptr, w ? w->data_ptr() : nullptr,
                               T, ns, W, static_cast<float>(eps), dt, cur_stream()),
        "hyper_update_norm");
}

void token_shift(at::Tensor out, const at::Tensor& n, const at::Tensor& mu, at::Tensor state,
                 const at::Tensor& positions, const at::Tensor& seq_qstart,
                 const at::Tensor& seq_slot) {
  f32c(n, "n");
  f32c(mu, "mu");
  f32c(state, "state");
  TORCH_CHECK(n.dim() == 2, "token_shift: n [T, W]");
  const int64_t T = n.size(0), W = n.size(1);
  meta(positions, seq_qstart, seq_slot, T);
  TORCH_CHECK(out.is_cuda() && out.is_contiguous() && out.sizes() == n.sizes() &&
                  mu.numel() == W && state.dim() == 2 && state.size(1) == W,
              "token_shift: shapes");
  const at::DeviceGuard g(n.device());
  rc_ok(mixk_token_shift(out.data_ptr(), n.data_ptr<float>(), mu.data_ptr<float>(),
                         state.data_ptr<float>(), positions.data_ptr<int>(),
                         seq_qstart.data_ptr<int>(), seq_slot.data_ptr<int>(), T, seq_slot.numel(),
                         W, code(out), cur_stream()),
        "token_shift");
}

void gate_mul(at::Tensor out, const at::Tensor& a, const at::Tensor& gate, int64_t act) {
  rows2d(gate, out, "gate");
  rows2d(a, out, "a");
  TORCH_CHECK(out.is_cuda() && out.is_contiguous() && out.dim() == 2 && out.sizes() == a.sizes() &&
                  gate.sizes() == a.sizes() && act >= 0 && act <= 2,
              "gate_mul: shapes");
  const at::DeviceGuard g(a.device());
  rc_ok(mixk_gate_mul(out.data_ptr(), a.data_ptr(), a.stride(0), gate.data_ptr(), gate.stride(0),
                      a.size(0), a.size(1), act, code(out), cur_stream()),
        "gate_mul");
}

void gelu(at::Tensor out, const at::Tensor& x, bool tanh_form) {
  rows2d(x, out, "x");
  TORCH_CHECK(out.is_contiguous() && out.sizes() == x.sizes(), "gelu: out");
  const at::DeviceGuard g(x.device());
  rc_ok(mixk_gelu(out.data_ptr(), x.data_ptr(), x.stride(0), x.size(0), x.size(1), tanh_form,
                  code(x), cur_stream()),
        "gelu");
}

void mingru_scan(at::Tensor out, at::Tensor state, const at::Tensor& z, const at::Tensor& x,
                 const at::Tensor& gt, const at::Tensor& positions, const at::Tensor& seq_qstart,
                 const at::Tensor& seq_slot) {
  rows2d(z, out, "z");
  rows2d(x, out, "x");
  rows2d(gt, out, "g");
  f32c(state, "state");
  const int64_t T = z.size(0), C = z.size(1), S = seq_slot.numel();
  meta(positions, seq_qstart, seq_slot, T);
  TORCH_CHECK(out.is_contiguous() && out.size(0) == T && out.size(1) == C && x.sizes() == z.sizes() &&
                  gt.sizes() == z.sizes() && state.dim() >= 2 && state.numel() == state.size(0) * C,
              "mingru_scan: shapes");
  const at::DeviceGuard g(z.device());
  rc_ok(mixk_mingru_scan(out.data_ptr(), state.data_ptr<float>(), z.data_ptr(), z.stride(0),
                         x.data_ptr(), x.stride(0), gt.data_ptr(), gt.stride(0),
                         positions.data_ptr<int>(), seq_qstart.data_ptr<int>(),
                         seq_slot.data_ptr<int>(), S, C, T <= 4 * S, code(out), cur_stream()),
        "mingru_scan");
}

void moe_route(at::Tensor idx, at::Tensor wts, const at::Tensor& logits, bool softmax,
               const c10::optional<at::Tensor>& correction, int64_t groups, int64_t keep,
               bool renorm) {
  f32c(logits, "logits");
  if (correction) {
    f32c(*correction, "correction");
    TORCH_CHECK(logits.dim() == 2 && correction->numel() == logits.size(1),
                "moe_route: correction [E]");
  }
  TORCH_CHECK(logits.dim() == 2 && groups >= 1 && logits.size(1) % groups == 0 && keep >= 1 &&
                  keep <= groups && idx.dim() == 2 &&
                  idx.size(1) <= keep * (logits.size(1) / groups),
              "moe_route: groups must split the experts evenly and the kept ones hold `top`");
  f32c(wts, "wts");
  i32(idx, "idx");
  TORCH_CHECK(logits.dim() == 2 && idx.dim() == 2 && idx.size(0) == logits.size(0) &&
                  wts.sizes() == idx.sizes() && idx.size(1) >= 1 && idx.size(1) <= logits.size(1),
              "moe_route: logits [T, E], idx / wts [T, top]");
  const at::DeviceGuard g(logits.device());
  rc_ok(mixk_moe_route(idx.data_ptr<int>(), wts.data_ptr<float>(), logits.data_ptr<float>(),
                       correction ? correction->data_ptr<float>() : nullptr, logits.size(0),
                       logits.size(1), idx.size(1), softmax, groups, keep, renorm, cur_stream()),
        "moe_route");
}

void moe_experts(at::Tensor y, at::Tensor act, at::Tensor plan, const at::Tensor& h,
                 const at::Tensor& idx, const at::Tensor& wts, const at::Tensor& w_gate,
                 const at::Tensor& w_up, const at::Tensor& w_down, double limit, double alpha,
                 int64_t max_tiles, int64_t tile_rows, int64_t split, int64_t glu) {
  i32(idx, "idx");
  i32(plan, "plan");
  f32c(wts, "wts");
  TORCH_CHECK(h.is_cuda() && h.dim() == 2 && h.is_contiguous() && idx.dim() == 2 &&
                  idx.size(0) == h.size(0) && wts.sizes() == idx.sizes() && w_gate.dim() == 3 &&
                  w_down.is_contiguous() && w_up.sizes() == w_gate.sizes() && w_down.dim() == 3 &&
                  w_gate.stride(2) == 1 && w_gate.stride(1) == w_gate.size(2) &&
                  w_up.strides() == w_gate.strides() && w_gate.stride(0) % 8 == 0,
              "moe_experts: h [T, W], idx / wts [T, top], w_gate / w_up [E, ff, W]");
  const int64_t T = h.size(0), W = h.size(1), top = idx.size(1), E = w_gate.size(0);
  const int64_t ff = w_gate.size(1), P = T * top;
  TORCH_CHECK(w_gate.size(2) == W && w_down.size(0) == E && w_down.size(1) == W &&
                  w_down.size(2) == ff && y.is_contiguous() && y.dim() == 2 && split >= 1 &&
                  split <= 64 && y.size(0) == P * split && y.size(1) == W && act.is_contiguous() && act.dim() == 2 && act.size(0) == P &&
                  act.size(1) == ff && plan.numel() >= 2 + 3 * max_tiles + P &&
                  (tile_rows == 64 || tile_rows == 128) &&
                  max_tiles >= P / tile_rows + std::min(E, P) && P < (int64_t{1} << 30) &&
                  w_gate.scalar_type() == h.scalar_type() && w_up.scalar_type() == h.scalar_type() &&
                  w_down.scalar_type() == h.scalar_type() &&
                  y.scalar_type() == (split > 1 ? at::kFloat : h.scalar_type()) &&
                  act.scalar_type() == h.scalar_type(),
              "moe_experts: shapes");
  const at::DeviceGuard g(h.device());
  rc_ok(mixk_moe_experts(y.data_ptr(), act.data_ptr(), plan.data_ptr<int>(), h.data_ptr(),
                         idx.data_ptr<int>(), wts.data_ptr<float>(), w_gate.data_ptr(),
                         w_up.data_ptr(), w_down.data_ptr(), T, top, E, ff, W, w_gate.stride(0), max_tiles,
                         tile_rows, split,
                         static_cast<float>(limit), static_cast<float>(alpha), glu, code(h),
                         cur_stream()),
        "moe_experts");
}

void pair_sum(at::Tensor out, const at::Tensor& y) {
  TORCH_CHECK(y.is_cuda() && y.dim() == 3 && y.is_contiguous() && out.is_cuda() &&
                  out.is_contiguous() && out.dim() == 2 && out.size(0) == y.size(0) &&
                  out.size(1) == y.size(2) &&
                  (out.scalar_type() == y.scalar_type() || y.scalar_type() == at::kFloat),
              "pair_sum: y [T, top, W] (out's dtype or fp32), out [T, W]");
  const at::DeviceGuard g(y.device());
  rc_ok(mixk_pair_sum(out.data_ptr(), y.data_ptr(), y.scalar_type() == at::kFloat, y.size(0),
                      y.size(1), y.size(2), code(out), cur_stream()),
        "pair_sum");
}

void clamped_glu(at::Tensor out, const at::Tensor& gu, const at::Tensor& wts, double limit,
                 double alpha) {
  f32c(wts, "wts");
  TORCH_CHECK(gu.is_cuda() && gu.dim() == 2 && gu.is_contiguous() && gu.size(1) % 2 == 0 &&
                  out.is_cuda() && out.is_contiguous() && out.dim() == 2 &&
                  out.size(0) == gu.size(0) && out.size(1) * 2 == gu.size(1) &&
                  wts.numel() == gu.size(0) && out.scalar_type() == gu.scalar_type(),
              "clamped_glu: gu [R, 2 ff], out [R, ff], wts [R]");
  const at::DeviceGuard g(gu.device());
  rc_ok(mixk_clamped_glu(out.data_ptr(), gu.data_ptr(), wts.data_ptr<float>(), gu.size(0),
                         out.size(1), static_cast<float>(limit), static_cast<float>(alpha),
                         code(gu), cur_stream()),
        "clamped_glu");
}

void moe_combine(at::Tensor out, const at::Tensor& y, const at::Tensor& idx, const at::Tensor& wts,
                 const at::Tensor& h, const c10::optional<at::Tensor>& addend, int64_t E,
                 int64_t split) {
  i32(idx, "idx");
  f32c(wts, "wts");
  TORCH_CHECK(h.is_cuda() && h.dim() == 2 && h.is_contiguous() && out.is_cuda() &&
                  out.is_contiguous() && out.sizes() == h.sizes() &&
                  out.scalar_type() == h.scalar_type() && idx.dim() == 2 &&
                  idx.size(0) == h.size(0) && wts.sizes() == idx.sizes() && split >= 1 &&
                  y.is_cuda() && y.is_contiguous() && y.dim() == 2 &&
                  y.size(0) == h.size(0) * idx.size(1) * split && y.size(1) == h.size(1) &&
                  (y.scalar_type() == h.scalar_type() || y.scalar_type() == at::kFloat) && E >= 0,
              "moe_combine: h / out [T, W], idx / wts [T, top], y [T * top * split, W]");
  if (addend)
    TORCH_CHECK(addend->is_cuda() && addend->is_contiguous() && addend->sizes() == h.sizes() &&
                    addend->scalar_type() == h.scalar_type(),
                "moe_combine: addend [T, W]");
  const at::DeviceGuard g(h.device());
  rc_ok(mixk_moe_combine(out.data_ptr(), y.data_ptr(), y.scalar_type() == at::kFloat,
                         idx.data_ptr<int>(), wts.data_ptr<float>(), h.data_ptr(),
                         addend ? addend->data_ptr() : nullptr, h.size(0), idx.size(1), split, E,
                         h.size(1), code(h), cur_stream()),
        "moe_combine");
}

void norm_add_norm(const c10::optional<at::Tensor>& h, at::Tensor x,
                   const c10::optional<at::Tensor>& y, const c10::optional<at::Tensor>& w_post,
                   const c10::optional<at::Tensor>& w_next, double eps, bool layer) {
  f32c(x, "x");
  TORCH_CHECK(x.dim() == 2 && (h.has_value() || y.has_value()) &&
                  h.has_value() == w_next.has_value() && y.has_value() == w_post.has_value(),
              "norm_add_norm: x [T, W]; y with w_post, h with w_next");
  const at::Tensor& like = h ? *h : *y;
  auto rows = [&](const at::Tensor& t) {
    TORCH_CHECK(t.is_cuda() && t.is_contiguous() && t.sizes() == x.sizes() &&
                    t.scalar_type() == like.scalar_type(),
                "norm_add_norm: rows [T, W] of one activation dtype");
  };
  auto weight = [&](const at::Tensor& t) {
    TORCH_CHECK(t.is_cuda() && t.is_contiguous() && t.numel() == x.size(1) &&
                    t.scalar_type() == like.scalar_type(),
                "norm_add_norm: weights [W] of the activation dtype");
  };
  if (h) { rows(*h); weight(*w_next); }
  if (y) { rows(*y); weight(*w_post); }
  const at::DeviceGuard g(x.device());
  rc_ok(mixk_norm_add_norm(h ? h->data_ptr() : nullptr, x.data_ptr<float>(),
                           y ? y->data_ptr() : nullptr, w_post ? w_post->data_ptr() : nullptr,
                           w_next ? w_next->data_ptr() : nullptr, x.size(0), x.size(1),
                           static_cast<float>(eps), layer, code(like), cur_stream()),
        "norm_add_norm");
}

void proj_inv_rms(at::Tensor out, const at::Tensor& qx, const at::Tensor& kx, double eps) {
  f32c(out, "out");
  rows2d(qx, qx, "q");
  rows2d(kx, qx, "k");
  TORCH_CHECK(out.numel() == 2 * qx.size(0) && kx.size(0) == qx.size(0) && qx.size(1) > 0 &&
                  kx.size(1) > 0,
              "proj_inv_rms: out [T, 2], q [T, nq], k [T, nk]");
  const at::DeviceGuard g(qx.device());
  rc_ok(mixk_proj_inv_rms(out.data_ptr<float>(), qx.data_ptr(), qx.stride(0), qx.size(1),
                          kx.data_ptr(), kx.stride(0), kx.size(1), qx.size(0),
                          static_cast<float>(eps), code(qx), cur_stream()),
        "proj_inv_rms");
}

void scale_softcap(at::Tensor out, const at::Tensor& logits, double scale, double cap) {
  f32c(out, "out");
  TORCH_CHECK(logits.is_cuda() && logits.is_contiguous() && out.sizes() == logits.sizes() &&
                  cap >= 0.0,
              "scale_softcap: contiguous logits, fp32 out of the same shape");
  const at::DeviceGuard g(logits.device());
  rc_ok(mixk_scale_softcap(out.data_ptr<float>(), logits.data_ptr(), logits.numel(),
                           static_cast<float>(scale), static_cast<float>(cap), code(logits),
                           cur_stream()),
        "scale_softcap");
}

}  // namespace

TORCH_LIBRARY(atta_mix, m) {
  m.def("embed_pair(Tensor(a!) out, Tensor table, Tensor pair_table, Tensor ids, Tensor positions, "
        "Tensor seq_qstart, Tensor seq_slot, Tensor(b!) prev_token, int mul_prev, int mul_cur, "
        "int buckets) -> ()");
  m.def("rms_norm_f32(Tensor(a!) out, Tensor x, Tensor w, float eps, bool one_plus) -> ()");
  m.def("relu_sq(Tensor(a!) out, Tensor x) -> ()");
  m.def("residual_add(Tensor(a!) x, Tensor a, float sa, Tensor? b, float sb, Tensor? c) -> ()");
  m.def("add_norm(Tensor(a!) h, Tensor(b!) x, Tensor a, float sa, Tensor? b, float sb, Tensor? c, "
        "Tensor w, float eps, bool one_plus) -> ()");
  m.def("gated_rms_norm(Tensor(a!) out, Tensor o, Tensor gate, Tensor w, float eps, int act) -> ()");
  m.def("qk_norm_rope_cache(Tensor(a!) q_out, Tensor qx, Tensor kx, Tensor vx, Tensor? q_norm, "
        "Tensor? k_norm, float eps, Tensor positions, Tensor slot_mapping, Tensor cos_sin, "
        "Tensor(b!) k_cache, Tensor(c!) v_cache, bool rotate_half, bool norm_last, "
        "Tensor? row_inv) -> ()");
  m.def("rotary_table(Tensor(a!) out, Tensor positions, Tensor inv_freq) -> ()");
  m.def("sink_attention(Tensor(a!) out, Tensor q, Tensor k_cache, Tensor v_cache, "
        "Tensor block_tables, Tensor seq_kvlen, Tensor seq_qstart, Tensor tile_seq, "
        "Tensor tile_qoff, float scale, bool sink, int num_decode, int max_decode_kv, "
        "Tensor? part, bool use_mfma, Tensor? sink_val, int window) -> ()");
  m.def("short_conv_silu(Tensor(a!) out, Tensor x, Tensor w, Tensor(b!) conv_state, "
        "Tensor positions, Tensor seq_qstart, Tensor seq_slot, Tensor? bias) -> ()");
  m.def("gated_delta_rule(Tensor(a!) out, Tensor qkv, Tensor beta, Tensor decay, Tensor a_log, "
        "Tensor dt_bias, Tensor(b!) state, Tensor positions, Tensor seq_qstart, Tensor seq_slot, "
        "int H, int G, int dim, int vdim) -> ()");
  m.def("embed_scale(Tensor(a!) out, Tensor table, Tensor ids, float scale) -> ()");
  m.def("rms_norm_rows(Tensor(a!) out, Tensor x, Tensor w, float eps) -> ()");
  m.def("xielu_bias(Tensor(a!) out, Tensor x, Tensor? bias, float ap, float aq) -> ()");
  m.def("group_rms_norm(Tensor(a!) out, Tensor y, Tensor? gate, Tensor w, int n_groups, float eps) "
        "-> ()");
  m.def("head_gate(Tensor(a!) out, Tensor o, Tensor gate) -> ()");
  m.def("latent_rope_cache(Tensor(a!) q_out, Tensor q_lat, Tensor qx, Tensor? kvx, Tensor? c_norm, "
        "float eps, Tensor slot_mapping, Tensor cos_sin, Tensor(b!) k_cache, Tensor(c!) v_cache, "
        "Tensor(d!) c_out) -> ()");
  m.def("gated_linear_scan(Tensor(a!) out, Tensor(b!) state, Tensor q, Tensor k, Tensor v, "
        "Tensor? dt, Tensor p0, Tensor p1, Tensor? p2, Tensor positions, Tensor seq_qstart, "
        "Tensor seq_slot, int H, int G, int dk, int dv, int mode) -> ()");
  m.def("hyper_update_norm(Tensor(a!)? out, Tensor(b!) xs, Tensor? y, Tensor? mix, Tensor? w_out, "
        "Tensor? w_in, Tensor? w, float eps) -> ()");
  m.def("token_shift(Tensor(a!) out, Tensor n, Tensor mu, Tensor(b!) state, Tensor positions, "
        "Tensor seq_qstart, Tensor seq_slot) -> ()");
  m.def("gate_mul(Tensor(a!) out, Tensor a, Tensor gate, int act) -> ()");
  m.def("gelu(Tensor(a!) out, Tensor x, bool tanh_form) -> ()");
  m.def("mingru_scan(Tensor(a!) out, Tensor(b!) state, Tensor z, Tensor x, Tensor g, "
        "Tensor positions, Tensor seq_qstart, Tensor seq_slot) -> ()");
  m.def("pair_sum(Tensor(a!) out, Tensor y) -> ()");
  m.def("clamped_glu(Tensor(a!) out, Tensor gu, Tensor wts, float limit, float alpha) -> ()");
  m.def("moe_route(Tensor(a!) idx, Tensor(b!) wts, Tensor logits, bool softmax, Tensor? correction, "
        "int groups, int keep, bool renorm) -> ()");
  m.def("moe_experts(Tensor(a!) y, Tensor(b!) act, Tensor(c!) plan, Tensor h, Tensor idx, "
        "Tensor wts, Tensor w_gate, Tensor w_up, Tensor w_down, float limit, float alpha, "
        "int max_tiles, int tile_rows, int split, int glu) -> ()");
  m.def("moe_combine(Tensor(a!) out, Tensor y, Tensor idx, Tensor wts, Tensor h, Tensor? addend, "
        "int E, int split) -> ()");
  m.def("norm_add_norm(Tensor(a!)? h, Tensor(b!) x, Tensor? y, Tensor? w_post, Tensor? w_next, "
        "float eps, bool layer) -> ()");
  m.def("proj_inv_rms(Tensor(a!) out, Tensor qx, Tensor kx, float eps) -> ()");
  m.def("scale_softcap(Tensor(a!) out, Tensor logits, float scale, float cap) -> ()");
}

TORCH_LIBRARY_IMPL(atta_mix, CUDA, m) {
  m.impl("embed_pair", &embed_pair);
  m.impl("rms_norm_f32", &rms_norm_f32);
  m.impl("relu_sq", &relu_sq);
  m.impl("residual_add", &residual_add);
  m.impl("add_norm", &add_norm);
  m.impl("gated_rms_norm", &gated_rms_norm);
  m.impl("qk_norm_rope_cache", &qk_norm_rope_cache);
  m.impl("rotary_table", &rotary_table);
  m.impl("sink_attention", &sink_attention);
  m.impl("short_conv_silu", &short_conv_silu);
  m.impl("gated_delta_rule", &gated_delta_rule);
  m.impl("embed_scale", &embed_scale);
  m.impl("rms_norm_rows", &rms_norm_rows);
  m.impl("xielu_bias", &xielu_bias);
  m.impl("group_rms_norm", &group_rms_norm);
  m.impl("head_gate", &head_gate);
  m.impl("latent_rope_cache", &latent_rope_cache);
  m.impl("gated_linear_scan", &gated_linear_scan);
  m.impl("hyper_update_norm", &hyper_update_norm);
  m.impl("token_shift", &token_shift);
  m.impl("gate_mul", &gate_mul);
  m.impl("gelu", &gelu);
  m.impl("mingru_scan", &mingru_scan);
  m.impl("pair_sum", &pair_sum);
  m.impl("clamped_glu", &clamped_glu);
  m.impl("moe_route", &moe_route);
  m.impl("moe_experts", &moe_experts);
  m.impl("moe_combine", &moe_combine);
  m.impl("norm_add_norm", &norm_add_norm);
  m.impl("proj_inv_rms", &proj_inv_rms);
  m.impl("scale_softcap", &scale_softcap);
}
