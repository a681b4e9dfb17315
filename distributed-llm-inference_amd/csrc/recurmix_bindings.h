// torch.ops.dli.rm_* — argument checks around the launchers of kernels/recurmix.hip (gated linear recurrences, gated latent
// attention).  Included by torch_bindings.cpp inside its anonymous namespace, after hypermix_bindings.h (uses the helpers of
// the earlier binding headers).  Every shape the kernels index with is checked here: the kernels themselves do no bounds checks.
#pragma once

const double* rot_freq(const Tensor& freq, int64_t rot_dims) {
  TORCH_CHECK(freq.is_cuda() && freq.scalar_type() == at::kDouble && freq.is_contiguous() && freq.numel() >= rot_dims / 2,
              "freq must be a float64 GPU tensor [rot_dims / 2]");
  return freq.data_ptr<double>();
}

// x [T, C] (row-strided view) → bias + Σ_j w[j] · x[t - taps + 1 + j] within each sequence; state [slots, taps-1, C] fp32 moves on
Tensor rm_causal_conv(const Tensor& x, const Tensor& w, const c10::optional<Tensor>& bias, Tensor state, const Tensor& positions,
                      const Tensor& token_seq, const Tensor& qsl, const Tensor& state_slots, const Tensor& counts, int64_t num_seqs,
                      bool out_bf16) {
  const bool bf = act_bf16(x, "x");
  check_rows(x, "x");
  const int64_t T = x.size(0), C = x.size(1);
  check_f32(w, "w");
  TORCH_CHECK(w.dim() == 2 && w.size(1) == C && w.size(0) >= 1 && w.size(0) <= dli::rm_max_taps(), "w must be [taps, C], taps in 1..",
              dli::rm_max_taps());
  const int64_t taps = w.size(0);
  const float* bp = opt_f32(bias, "bias", C);
  check_f32(state, "state");
  TORCH_CHECK(state.dim() == 3 && state.size(1) == taps - 1 && state.size(2) == C, "state must be [slots, taps-1, C]");
  check_i32(token_seq, "token_seq");
  TORCH_CHECK(token_seq.numel() >= T, "token_seq shorter than the batch");
  check_step_meta(positions, qsl, state_slots, counts, T, num_seqs);
  Tensor out = at::empty({T, C}, x.options().dtype(out_bf16 ? at::kBFloat16 : at::kFloat));
  dli::launch_rm_causal_conv(x.data_ptr(), bf, x.stride(0), w.data_ptr<float>(), bp, (int)taps, state.data_ptr<float>(),
                             positions.data_ptr<int>(), token_seq.data_ptr<int>(), qsl.data_ptr<int>(), state_slots.data_ptr<int>(),
                             counts.data_ptr<int>(), (int)T, (int)num_seqs, (int)C, out.data_ptr(), out_bf16, cur_stream(x));
  return out;
}

// z [B, T, 2n] gate pre-activations, u [T, B·n], y [T, B·n] (row-strided view), gate_bias fp32 [2, B·n], rate fp32 [B·n],
// state fp32 [slots, B·n] → S · gelu_tanh(y), rows of padding zero
Tensor rm_rglru_scan(const Tensor& z, const Tensor& u, const Tensor& y, const Tensor& gate_bias, const Tensor& rate, Tensor state,
                     const Tensor& positions, const Tensor& qsl, const Tensor& state_slots, const Tensor& counts, int64_t num_seqs,
                     bool out_bf16, const c10::optional<Tensor>& tile_seq, const c10::optional<Tensor>& tile_q0, int64_t num_tiles) {
  const bool bf = act_bf16(u, "u");
  check_act_like(z, bf, "z");
  check_act_like(y, bf, "y");
  TORCH_CHECK(z.dim() == 3 && z.is_contiguous() && z.size(2) % 2 == 0, "z must be contiguous [B, T, 2n]");
  const int64_t B = z.size(0), T = z.size(1), n = z.size(2) / 2, C = B * n;
  TORCH_CHECK(u.dim() == 2 && u.is_contiguous() && u.size(0) == T && u.size(1) == C, "u must be contiguous [T, B·n]");
  check_rows(y, "y");
  TORCH_CHECK(y.size(0) == T && y.size(1) == C, "y must be [T, B·n]");
  check_f32(gate_bias, "gate_bias", 2 * C);
  check_f32(rate, "rate", C);
  check_f32(state, "state");
  TORCH_CHECK(state.dim() == 2 && state.size(1) == C, "state must be [slots, B·n]");
  check_step_meta(positions, qsl, state_slots, counts, T, num_seqs);
  Tensor out = at::zeros({T, C}, u.options().dtype(out_bf16 ? at::kBFloat16 : at::kFloat));
  // chunks of two tokens or more run block-parallel over the step's 64-token tiles when the caller hands them in
  const int* tsp = nullptr;
  const int* tqp = nullptr;
  Tensor ws;
  if (num_tiles > 0 && tile_seq.has_value() && tile_q0.has_value()) {
    check_i32(*tile_seq, "tile_seq");
    check_i32(*tile_q0, "tile_q0");
    TORCH_CHECK(tile_seq->numel() >= num_tiles && tile_q0->numel() >= num_tiles, "tile lists shorter than num_tiles");
    tsp = tile_seq->data_ptr<int>();
    tqp = tile_q0->data_ptr<int>();
    ws = at::empty({dli::rm_rglru_ws_floats((int)T, (int)num_seqs, (int)C)}, u.options().dtype(at::kFloat));
  } else {
    num_tiles = 0;
  }
  dli::launch_rm_rglru_scan(z.data_ptr(), u.data_ptr(), y.data_ptr(), bf, y.stride(0), gate_bias.data_ptr<float>(), rate.data_ptr<float>(),
                            state.data_ptr<float>(), positions.data_ptr<int>(), qsl.data_ptr<int>(), state_slots.data_ptr<int>(),
                            counts.data_ptr<int>(), (int)T, (int)num_seqs, (int)B, (int)n, out.data_ptr(), out_bf16, tsp, tqp, (int)num_tiles,
                            num_tiles > 0 ? ws.data_ptr<float>() : nullptr, cur_stream(u));
  return out;
}

// leading columns of proj rows = [query latent (Q) | key / value latent (C) | shared key part (R)]; returns the normed query
// latent [T, Q]; with a cache [pages, page tokens, C + R] the normed latent and the rotated key part go to the rows slot_mapping
Tensor rm_latent_norm_cache(const Tensor& proj, int64_t Q, const Tensor& qw, const c10::optional<Tensor>& cw, double eps,
                            const Tensor& positions, const Tensor& freq, double mag, int64_t rot_dims, const Tensor& slot_mapping,
                            const c10::optional<Tensor>& cache, int64_t C, int64_t R) {
  const bool bf = act_bf16(proj, "proj");
  check_rows(proj, "proj");
  const int64_t T = proj.size(0);
  TORCH_CHECK(Q > 0 && C > 0 && R >= 0, "latent sizes must be positive");
  check_f32(qw, "qw", Q);
  TORCH_CHECK(rot_dims >= 0 && rot_dims % 2 == 0 && rot_dims <= R && rot_dims * 4 <= kSmMaxLds, "rot_dims must be even and at most R");
  check_i32(positions, "positions");
  check_i32(slot_mapping, "slot_mapping");
  TORCH_CHECK(positions.numel() >= T && slot_mapping.numel() >= T, "step metadata shorter than the batch");
  Tensor cq = at::empty({T, Q}, proj.options());
  void* cp = nullptr;
  const float* cwp = nullptr;
  const double* fp = nullptr;
  if (cache.has_value()) {
    TORCH_CHECK(proj.size(1) >= Q + C + R, "proj rows shorter than the three parts");
    check_act_like(*cache, bf, "cache");
    TORCH_CHECK(cache->is_contiguous() && cache->dim() == 3 && cache->size(1) == kSmPageTokens && cache->size(2) == C + R,
                "cache must be contiguous [pages, page tokens, C + R]");
    TORCH_CHECK(cw.has_value(), "a cache needs the latent's norm weight");
    check_f32(*cw, "cw", C);
    cwp = cw->data_ptr<float>();
    cp = cache->data_ptr();
    if (rot_dims > 0) fp = rot_freq(freq, rot_dims);
  } else {
    TORCH_CHECK(proj.size(1) >= Q, "proj rows shorter than the query latent");
  }
  dli::launch_rm_latent_norm_cache(proj.data_ptr(), bf, proj.stride(0), (int)Q, qw.data_ptr<float>(), cwp, (float)eps,
                                   positions.data_ptr<int>(), fp, (float)mag, (int)rot_dims, slot_mapping.data_ptr<int>(), cp, (int)T,
                                   (int)C, (int)R, cq.data_ptr(), cur_stream(proj));
  return cq;
}

void rm_rotate_heads(Tensor q, const Tensor& positions, const Tensor& freq, double mag, int64_t rot_dims, int64_t H, int64_t D, int64_t R) {
  const bool bf = act_bf16(q, "q");
  check_rows(q, "q");
  const int64_t T = q.size(0);
  TORCH_CHECK(H > 0 && D >= 0 && R >= 0 && q.size(1) >= H * (D + R), "q rows shorter than H heads of D + R");
  TORCH_CHECK(rot_dims >= 0 && rot_dims % 2 == 0 && rot_dims <= R && rot_dims * 4 <= kSmMaxLds, "rot_dims must be even and at most R");
  check_i32(positions, "positions");
  TORCH_CHECK(positions.numel() >= T, "positions shorter than the batch");
  if (rot_dims == 0) return;
  dli::launch_rm_rotate_heads(q.data_ptr(), bf, q.stride(0), positions.data_ptr<int>(), rot_freq(freq, rot_dims), (float)mag,
                              (int)rot_dims, (int)T, (int)H, (int)D, (int)R, cur_stream(q));
}

// o [H, T, Dv] · sigmoid(gate [T, H·Dv] (row-strided view)) → [T, H·Dv]
Tensor rm_gate_heads(const Tensor& o, const Tensor& gate) {
  const bool bf = act_bf16(o, "o");
  TORCH_CHECK(o.dim() == 3 && o.is_contiguous(), "o must be contiguous [H, T, Dv]");
  const int64_t H = o.size(0), T = o.size(1), Dv = o.size(2);
  check_act_like(gate, bf, "gate");
  check_rows(gate, "gate");
  TORCH_CHECK(gate.size(0) == T && gate.size(1) == H * Dv, "gate must be [T, H·Dv]");
  Tensor out = at::empty({T, H * Dv}, o.options());
  dli::launch_rm_gate_heads(o.data_ptr(), gate.data_ptr(), bf, gate.stride(0), (int)H, (int)T, (int)Dv, out.data_ptr(), cur_stream(o));
  return out;
}

// clamped gated experts; an id outside 0..E-1 names an identity expert (its output is the input row)
Tensor rm_clamped_experts(const Tensor& h, const Tensor& ids, const Tensor& wts, const Tensor& gate_up, const Tensor& down, double limit) {
  const bool bf = act_bf16(h, "h");
  check_rows(h, "h");
  const int64_t T = h.size(0), W = h.size(1);
  check_act_like(gate_up, bf, "gate_up");
  check_act_like(down, bf, "down");
  TORCH_CHECK(gate_up.dim() == 3 && down.dim() == 3 && gate_up.is_contiguous() && down.is_contiguous(), "expert weights must be contiguous 3-D");
  const int64_t E = gate_up.size(0), F = gate_up.size(1) / 2;
  TORCH_CHECK(gate_up.size(1) == 2 * F && gate_up.size(2) == W && down.size(0) == E && down.size(1) == W && down.size(2) == F,
              "expert weights must be [E, 2F, W] and [E, W, F]");
  TORCH_CHECK(limit > 0.0, "the clamp needs a positive limit");
  check_i32(ids, "ids");
  check_f32(wts, "wts");
  TORCH_CHECK(ids.dim() == 2 && ids.size(0) == T && wts.dim() == 2 && wts.size(0) == T && wts.size(1) == ids.size(1), "ids / wts must be [T, K]");
  const int64_t K = ids.size(1);
  Tensor out = at::empty({T, W}, h.options());
  if (bf && g_dm_grouped_experts && W % 128 == 0 && F % 64 == 0 && E <= 64 && (T * K >= 64 || F % 128 == 0) && h.is_contiguous() &&
      reinterpret_cast<uintptr_t>(h.data_ptr()) % 16 == 0) {
    // the expert kernels of the Mixtral path (weight streaming at decode size, else grouped GEMMs) with the clamped activation
    // in their first epilogue; pairs of identity experts are outside the expert range and skipped there
    moe_apply(h, ids, wts, gate_up, down, K, 0, E, 0, out, cur_stream(h), (float)limit);
    dli::launch_rm_identity_add(out.data_ptr(), h.data_ptr(), bf, h.stride(0), ids.data_ptr<int>(), wts.data_ptr<float>(), (int)K, (int)E,
                                (int)T, (int)W, cur_stream(h));
    return out;
  }
  TORCH_CHECK(W * 4 <= kSmMaxLds && K * F * 4 <= kSmMaxLds, "rows too wide");
  Tensor act = at::empty({T * K, F}, h.options());
  dli::launch_dm_experts(h.data_ptr(), bf, h.stride(0), ids.data_ptr<int>(), wts.data_ptr<float>(), (int)K, gate_up.data_ptr(),
                         down.data_ptr(), (int)T, (int)F, (int)W, act.data_ptr(), out.data_ptr(), 2, (int)E, (float)limit, cur_stream(h));
  return out;
}
