// torch.ops.dli.hm_* — argument checks around the launchers of kernels/hypermix.hip (hyper-connected stacks).
// Included by torch_bindings.cpp inside its anonymous namespace, after dualmix_bindings.h (uses the helpers of both).
// Every shape the kernels index with is checked here: the kernels themselves do no bounds checks.
#pragma once

// x [T, S, W] fp32, updated in place when y is given; returns the normed read [T, W] (empty without in_w)
Tensor hm_stream_mix_norm(Tensor x, const c10::optional<Tensor>& y, const c10::optional<Tensor>& mix, const c10::optional<Tensor>& out_w,
                          const c10::optional<Tensor>& in_w, const c10::optional<Tensor>& norm_w, double eps, double w_offset,
                          bool out_bf16, bool center) {
  check_f32(x, "x");
  TORCH_CHECK(x.dim() == 3, "x must be [T, S, W]");
  const int64_t T = x.size(0), S = x.size(1), W = x.size(2);
  TORCH_CHECK(S >= 1 && S <= dli::hm_max_streams(), "between 1 and ", dli::hm_max_streams(), " streams");
  TORCH_CHECK(y.has_value() == mix.has_value() && y.has_value() == out_w.has_value(), "y, mix and out_w come together");
  TORCH_CHECK(in_w.has_value() == norm_w.has_value(), "in_w and norm_w come together");
  const void* yp = nullptr;
  bool ybf = false;
  int64_t ys = 0;
  if (y.has_value()) {
    ybf = act_bf16(*y, "y");
    check_rows(*y, "y");
    TORCH_CHECK(y->size(0) == T && y->size(1) == W, "y must be [T, W]");
    yp = y->data_ptr();
    ys = y->stride(0);
  }
  const float* mp = opt_f32(mix, "mix", S * S);
  const float* op = opt_f32(out_w, "out_w", S);
  const float* ip = opt_f32(in_w, "in_w", S);
  const float* np = opt_f32(norm_w, "norm_w", W);
  TORCH_CHECK(W * 4 <= kSmMaxLds, "row too wide");
  Tensor out = at::empty({ip ? T : 0, W}, x.options().dtype(out_bf16 ? at::kBFloat16 : at::kFloat));
  dli::launch_hm_stream_mix_norm(x.data_ptr<float>(), yp, ybf, ys, mp, op, ip, np, (float)eps, (float)w_offset, (int)T, (int)S, (int)W,
                                 out.data_ptr(), out_bf16, center, cur_stream(x));
  return out;
}

Tensor hm_causal_conv_add(const Tensor& h, const Tensor& w, Tensor state, const Tensor& positions, const Tensor& token_seq,
                          const Tensor& qsl, const Tensor& state_slots, const Tensor& counts, int64_t num_seqs, bool out_bf16) {
  check_f32(h, "h");
  TORCH_CHECK(h.dim() == 2, "h must be [T, W]");
  const int64_t T = h.size(0), W = h.size(1);
  check_f32(w, "w");
  TORCH_CHECK(w.dim() == 2 && w.size(1) == W && w.size(0) >= 1 && w.size(0) <= dli::hm_max_taps(), "w must be [taps, W], taps in 1..",
              dli::hm_max_taps());
  const int64_t taps = w.size(0);
  check_f32(state, "state");
  if (taps > 1)
    TORCH_CHECK(state.dim() == 3 && state.size(1) == taps - 1 && state.size(2) == W, "state must be [slots, taps-1, W]");
  check_i32(token_seq, "token_seq");
  TORCH_CHECK(token_seq.numel() >= T, "token_seq shorter than the batch");
  check_step_meta(positions, qsl, state_slots, counts, T, num_seqs);
  Tensor out = at::empty({T, W}, h.options().dtype(out_bf16 ? at::kBFloat16 : at::kFloat));
  dli::launch_hm_causal_conv_add(h.data_ptr<float>(), w.data_ptr<float>(), (int)taps, state.data_ptr<float>(), positions.data_ptr<int>(),
                                 token_seq.data_ptr<int>(), qsl.data_ptr<int>(), state_slots.data_ptr<int>(), counts.data_ptr<int>(),
                                 (int)T, (int)num_seqs, (int)W, out.data_ptr(), out_bf16, cur_stream(h));
  return out;
}

Tensor hm_retention_prep(const Tensor& qkvg, const Tensor& positions, const c10::optional<Tensor>& freq, int64_t rot_dims, int64_t H,
                         int64_t D, int64_t Dv, double k_scale) {
  const bool bf = act_bf16(qkvg, "qkvg");
  check_rows(qkvg, "qkvg");
  const int64_t T = qkvg.size(0), n = 2 * H * D + H * Dv;
  TORCH_CHECK(H > 0 && D > 0 && Dv > 0 && qkvg.size(1) >= n, "qkvg rows shorter than q | k | v");
  TORCH_CHECK(rot_dims >= 0 && rot_dims % 2 == 0 && rot_dims <= D && rot_dims * 4 <= kSmMaxLds, "rot_dims must be even and at most D");
  const double* fp = nullptr;
  if (rot_dims > 0) {
    TORCH_CHECK(freq.has_value() && freq->is_cuda() && freq->scalar_type() == at::kDouble && freq->is_contiguous() &&
                    freq->numel() >= rot_dims / 2, "freq must be a float64 GPU tensor [rot_dims / 2]");
    fp = freq->data_ptr<double>();
  }
  check_i32(positions, "positions");
  TORCH_CHECK(positions.numel() >= T, "positions shorter than the batch");
  Tensor out = at::empty({T, n}, qkvg.options().dtype(at::kFloat));
  dli::launch_hm_retention_prep(qkvg.data_ptr(), bf, qkvg.stride(0), positions.data_ptr<int>(), fp, (int)rot_dims, (int)T, (int)H, (int)D,
                                (int)Dv, (float)k_scale, out.data_ptr<float>(), cur_stream(qkvg));
  return out;
}

Tensor hm_act_mul(const Tensor& x, bool silu) {
  const bool bf = act_bf16(x, "x");
  check_rows(x, "x");
  TORCH_CHECK(x.size(1) % 2 == 0, "rows must hold gate | up");
  const int64_t F = x.size(1) / 2;
  Tensor out = at::empty({x.size(0), F}, x.options());
  dli::launch_hm_act_mul(x.data_ptr(), bf, x.stride(0), (int)x.size(0), (int)F, silu, out.data_ptr(), cur_stream(x));
  return out;
}

// all: softmax over all logits, `bias` moves the choice only, weights renormalised over the chosen (rm_softmax_all_route)
std::tuple<Tensor, Tensor> hm_softmax_route(const Tensor& h, const Tensor& router, const c10::optional<Tensor>& bias, int64_t K,
                                            bool all) {
  const bool bf = act_bf16(h, "h");
  check_rows(h, "h");
  const int64_t T = h.size(0), W = h.size(1);
  check_f32(router, "router");
  TORCH_CHECK(router.dim() == 2 && router.size(1) == W, "router must be [E, W]");
  const int64_t E = router.size(0);
  TORCH_CHECK(E >= 1 && E <= 64 && K >= 1 && K <= E, "at most 64 experts, 1 <= top <= experts");
  const float* bp = opt_f32(bias, "bias", E);
  TORCH_CHECK(W * 4 <= kSmMaxLds, "row too wide");
  Tensor ids = at::empty({T, K}, h.options().dtype(at::kInt)), wts = at::empty({T, K}, h.options().dtype(at::kFloat));
  dli::launch_hm_softmax_route(h.data_ptr(), bf, h.stride(0), router.data_ptr<float>(), bp, (int)E, (int)K, (int)T, (int)W,
                               ids.data_ptr<int>(), wts.data_ptr<float>(), all, cur_stream(h));
  return {ids, wts};
}
