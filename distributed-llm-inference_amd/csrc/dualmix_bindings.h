// torch.ops.dli.dm_* — argument checks around the launchers of kernels/dualmix.hip (gated parallel layers).
// Included by torch_bindings.cpp inside its anonymous namespace, after seqmix_bindings.h (uses its helpers).
// Every shape the kernels index with is checked here: the kernels themselves do no bounds checks.
#pragma once

void check_act_like(const Tensor& t, bool bf16, const char* name) {
  TORCH_CHECK(act_bf16(t, name) == bf16, name, " must have the dtype of the other activations");
}
void check_step_meta(const Tensor& positions, const Tensor& qsl, const Tensor& state_slots, const Tensor& counts, int64_t T,
                     int64_t num_seqs) {
  check_i32(positions, "positions");
  check_i32(qsl, "query_start_loc");
  check_i32(state_slots, "state_slots");
  check_i32(counts, "counts");
  TORCH_CHECK(positions.numel() >= T && counts.numel() >= 4, "step metadata shorter than the batch");
  TORCH_CHECK(num_seqs >= 0 && qsl.numel() >= num_seqs + 1 && state_slots.numel() >= num_seqs, "batch-row metadata too short");
}

std::tuple<Tensor, Tensor> dm_rms_scale(const Tensor& x, const Tensor& g1, const c10::optional<Tensor>& g2, double eps, bool out_bf16) {
  check_f32(x, "x");
  TORCH_CHECK(x.dim() == 2, "x must be [rows, W]");
  check_f32(g1, "g1", 1);
  const float* g2p = opt_f32(g2, "g2", 1);
  auto opt = x.options().dtype(out_bf16 ? at::kBFloat16 : at::kFloat);
  Tensor h1 = at::empty({x.size(0), x.size(1)}, opt), h2 = at::empty({g2p ? x.size(0) : 0, x.size(1)}, opt);
  dli::launch_dm_rms_scale(x.data_ptr<float>(), g1.data_ptr<float>(), g2p, (float)eps, (int)x.size(0), (int)x.size(1), h1.data_ptr(),
                           h2.data_ptr(), out_bf16, cur_stream(x));
  return {h1, h2};
}

Tensor dm_shift_mix(const Tensor& h, const Tensor& mu, Tensor state, const Tensor& positions, const Tensor& token_seq, const Tensor& qsl,
                    const Tensor& state_slots, const Tensor& counts, int64_t num_seqs) {
  const bool bf = act_bf16(h, "h");
  check_rows(h, "h");
  const int64_t T = h.size(0), W = h.size(1);
  check_f32(mu, "mu");
  TORCH_CHECK(mu.dim() == 2 && mu.size(1) == W && mu.size(0) >= 1, "mu must be [S, W]");
  check_f32(state, "state");
  TORCH_CHECK(state.dim() == 2 && state.size(1) == W, "state must be [slots, W]");
  check_i32(token_seq, "token_seq");
  TORCH_CHECK(token_seq.numel() >= T, "token_seq shorter than the batch");
  check_step_meta(positions, qsl, state_slots, counts, T, num_seqs);
  Tensor out = at::empty({mu.size(0), T, W}, h.options());
  dli::launch_dm_shift_mix(h.data_ptr(), bf, h.stride(0), mu.data_ptr<float>(), (int)mu.size(0), state.data_ptr<float>(),
                           positions.data_ptr<int>(), token_seq.data_ptr<int>(), qsl.data_ptr<int>(), state_slots.data_ptr<int>(),
                           counts.data_ptr<int>(), (int)T, (int)num_seqs, (int)W, out.data_ptr(), cur_stream(h));
  return out;
}

// G = 0: the rows hold queries only (kw and both caches absent); rot_dims = 0: nothing is rotated (freq may be absent)
void dm_wide_norm_rope_cache(Tensor qkv, const Tensor& qw, const c10::optional<Tensor>& kw, double eps, const Tensor& positions,
                             const c10::optional<Tensor>& freq, double mag, int64_t rot_dims, const Tensor& slot_mapping,
                             const c10::optional<Tensor>& k_cache, const c10::optional<Tensor>& v_cache, int64_t H, int64_t G, int64_t D,
                             int64_t Dv) {
  const bool bf = act_bf16(qkv, "qkv");
  check_rows(qkv, "qkv");
  const int64_t T = qkv.size(0);
  TORCH_CHECK(H > 0 && G >= 0 && D > 0 && Dv > 0 && qkv.size(1) >= H * D + G * D + G * Dv, "qkv rows shorter than q | k | v");
  check_f32(qw, "qw", H * D);
  TORCH_CHECK((G > 0) == kw.has_value() && (G > 0) == k_cache.has_value() && (G > 0) == v_cache.has_value(),
              "key weights and both caches come with key / value heads, and only with them");
  const float* kwp = opt_f32(kw, "kw", G * D);
  TORCH_CHECK(rot_dims >= 0 && rot_dims % 2 == 0 && rot_dims <= D, "rot_dims must be even and at most D");
  TORCH_CHECK(rot_dims / 2 <= 256, "too many rotated pairs");
  const double* fp = nullptr;
  if (rot_dims > 0) {
    TORCH_CHECK(freq.has_value() && freq->is_cuda() && freq->scalar_type() == at::kDouble && freq->is_contiguous() &&
                    freq->numel() >= rot_dims / 2, "freq must be a float64 GPU tensor [rot_dims / 2]");
    fp = freq->data_ptr<double>();
  }
  check_i32(positions, "positions");
  check_i32(slot_mapping, "slot_mapping");
  TORCH_CHECK(positions.numel() >= T && slot_mapping.numel() >= T, "step metadata shorter than the batch");
  void* kp = nullptr;
  void* vp = nullptr;
  if (G > 0) {
    check_act_like(*k_cache, bf, "k_cache");
    check_act_like(*v_cache, bf, "v_cache");
    TORCH_CHECK(k_cache->is_contiguous() && v_cache->is_contiguous() && k_cache->dim() == 3 && v_cache->dim() == 3 &&
                    k_cache->size(1) == kSmPageTokens && v_cache->size(1) == kSmPageTokens && k_cache->size(2) == G * D &&
                    v_cache->size(2) == G * Dv && k_cache->size(0) == v_cache->size(0),
                "caches must be [pages, 32, G*D] and [pages, 32, G*Dv]");
    kp = k_cache->data_ptr();
    vp = v_cache->data_ptr();
  }
  TORCH_CHECK((H * D + G * D + rot_dims) * 4 <= kSmMaxLds, "q and k rows too wide");
  dli::launch_dm_wide_norm_rope_cache(qkv.data_ptr(), bf, qkv.stride(0), qw.data_ptr<float>(), kwp, (float)eps,
                                      positions.data_ptr<int>(), fp, (float)mag, (int)rot_dims, slot_mapping.data_ptr<int>(), kp, vp,
                                      (int)T, (int)H, (int)G, (int)D, (int)Dv, cur_stream(qkv));
}

void dm_talk_attention(Tensor out, const Tensor& q, const c10::optional<Tensor>& gate, const Tensor& k_cache, const Tensor& v_cache,
                       const Tensor& block_tables, const Tensor& positions, const Tensor& token_seq, const c10::optional<Tensor>& sink,
                       const c10::optional<Tensor>& talk, int64_t G, int64_t Dv, double scale, int64_t rows) {
  const bool bf = act_bf16(q, "q");
  TORCH_CHECK(q.dim() == 3 && q.stride(2) == 1, "q must be [T, H, D] with contiguous head rows");
  const int64_t T = q.size(0), H = q.size(1), D = q.size(2);
  TORCH_CHECK(rows <= T, "more rows than tokens");
  const int64_t todo = rows < 0 ? T : rows;                  // the leading rows this kernel serves (the tile kernel took the rest)
  TORCH_CHECK(G > 0 && H % G == 0 && Dv > 0, "heads must be a multiple of the key/value heads");
  check_act_like(out, bf, "out");
  check_rows(out, "out");
  TORCH_CHECK(out.size(0) == T && out.size(1) == H * Dv, "out must be [T, H*Dv]");
  const void* gp = nullptr;
  int64_t gs = 0;
  if (gate.has_value()) {
    check_act_like(*gate, bf, "gate");
    check_rows(*gate, "gate");
    TORCH_CHECK(gate->size(0) == T && gate->size(1) == H * Dv, "gate must be [T, H*Dv]");
    gp = gate->data_ptr();
    gs = gate->stride(0);
  }
  check_act_like(k_cache, bf, "k_cache");
  check_act_like(v_cache, bf, "v_cache");
  TORCH_CHECK(k_cache.is_contiguous() && v_cache.is_contiguous() && k_cache.dim() == 3 && v_cache.dim() == 3 &&
                  k_cache.size(1) == kSmPageTokens && v_cache.size(1) == kSmPageTokens && k_cache.size(2) == G * D &&
                  v_cache.size(2) == G * Dv && k_cache.size(0) == v_cache.size(0) && k_cache.size(0) * kSmPageTokens < (int64_t(1) << 31),
              "caches must be [pages, 32, G*D] and [pages, 32, G*Dv]");
  check_i32(block_tables, "block_tables");
  TORCH_CHECK(block_tables.dim() == 2, "block_tables must be [B, max_blocks]");
  check_i32(positions, "positions");
  check_i32(token_seq, "token_seq");
  TORCH_CHECK(positions.numel() >= T && token_seq.numel() >= T, "step metadata shorter than the batch");
  const float* sp = opt_f32(sink, "sink", H);
  const float* tp = opt_f32(talk, "talk", H * H);
  TORCH_CHECK(H <= dli::dm_talk_attention_max_heads() && H * Dv <= dli::dm_talk_attention_max_out(), "too many heads / output columns");
  TORCH_CHECK((int64_t)dli::dm_talk_attention_lds((int)H, (int)D) <= kSmMaxLds, "query rows too wide");
  dli::launch_dm_talk_attention(out.data_ptr(), out.stride(0), q.data_ptr(), q.stride(0), q.stride(1), gp, gs, k_cache.data_ptr(),
                                v_cache.data_ptr(), bf, block_tables.data_ptr<int>(), (int)block_tables.size(1), positions.data_ptr<int>(),
                                token_seq.data_ptr<int>(), sp, tp, (int)todo, (int)H, (int)G, (int)D, (int)Dv, (float)scale, cur_stream(q));
}

void dm_prepare() { dli::dm_prepare_kernels(); }

// prefill tiles of a bf16 step on the matrix cores; false: not covered (nothing was launched)
bool dm_talk_tile_attention(Tensor out, const Tensor& q, const c10::optional<Tensor>& gate, const Tensor& k_cache, const Tensor& v_cache,
                            const Tensor& block_tables, const Tensor& seq_lens, const Tensor& qsl, const Tensor& tile_seq,
                            const Tensor& tile_q0, int64_t num_tiles, const c10::optional<Tensor>& counts,
                            const c10::optional<Tensor>& sink, const c10::optional<Tensor>& talk, int64_t G, int64_t Dv, double scale) {
  if (!act_bf16(q, "q")) return false;
  TORCH_CHECK(q.dim() == 3 && q.stride(2) == 1, "q must be [T, H, D] with contiguous head rows");
  const int64_t T = q.size(0), H = q.size(1), D = q.size(2);
  TORCH_CHECK(G > 0 && H % G == 0 && Dv > 0, "heads must be a multiple of the key/value heads");
  check_act_like(out, true, "out");
  check_rows(out, "out");
  TORCH_CHECK(out.size(0) == T && out.size(1) == H * Dv, "out must be [T, H*Dv]");
  const void* gp = nullptr;
  int64_t gs = 0;
  if (gate.has_value()) {
    check_act_like(*gate, true, "gate");
    check_rows(*gate, "gate");
    TORCH_CHECK(gate->size(0) == T && gate->size(1) == H * Dv, "gate must be [T, H*Dv]");
    gp = gate->data_ptr();
    gs = gate->stride(0);
  }
  check_act_like(k_cache, true, "k_cache");
  check_act_like(v_cache, true, "v_cache");
  TORCH_CHECK(k_cache.is_contiguous() && v_cache.is_contiguous() && k_cache.dim() == 3 && v_cache.dim() == 3 &&
                  k_cache.size(1) == kSmPageTokens && v_cache.size(1) == kSmPageTokens && k_cache.size(2) == G * D &&
                  v_cache.size(2) == G * Dv && k_cache.size(0) == v_cache.size(0),
              "caches must be [pages, 32, G*D] and [pages, 32, G*Dv]");
  check_i32(block_tables, "block_tables");
  TORCH_CHECK(block_tables.dim() == 2, "block_tables must be [B, max_blocks]");
  check_i32(seq_lens, "seq_lens");
  check_i32(qsl, "query_start_loc");
  check_i32(tile_seq, "tile_seq");
  check_i32(tile_q0, "tile_q0");
  TORCH_CHECK(num_tiles >= 0 && tile_seq.numel() >= num_tiles && tile_q0.numel() >= num_tiles, "tile list shorter than num_tiles");
  TORCH_CHECK(qsl.numel() >= block_tables.size(0) + 1 && seq_lens.numel() >= block_tables.size(0), "batch-row metadata too short");
  const int* cnt = nullptr;
  if (counts.has_value()) {
    check_i32(*counts, "counts");
    TORCH_CHECK(counts->numel() >= 4, "counts too short");
    cnt = counts->data_ptr<int>();
  }
  return dli::launch_dm_talk_tile_attention(out.data_ptr(), out.stride(0), q.data_ptr(), q.stride(0), q.stride(1), gp, gs,
                                            k_cache.data_ptr(), v_cache.data_ptr(), block_tables.data_ptr<int>(),
                                            (int)block_tables.size(1), seq_lens.data_ptr<int>(), qsl.data_ptr<int>(),
                                            tile_seq.data_ptr<int>(), tile_q0.data_ptr<int>(), (int)num_tiles, cnt,
                                            opt_f32(sink, "sink", H), opt_f32(talk, "talk", H * H), (int)H, (int)G, (int)D, (int)Dv,
                                            (float)scale, cur_stream(q));
}

Tensor dm_decay(const Tensor& a, const Tensor& w2, const Tensor& w0) {
  const bool bf = act_bf16(a, "a");
  check_rows(a, "a");
  check_act_like(w2, bf, "w2");
  TORCH_CHECK(w2.dim() == 2 && w2.is_contiguous() && w2.size(1) == a.size(1), "w2 must be [C, L]");
  check_f32(w0, "w0", w2.size(0));
  TORCH_CHECK(a.size(1) * 4 <= kSmMaxLds, "rank too large");
  Tensor out = at::empty({a.size(0), w2.size(0)}, a.options().dtype(at::kFloat));
  dli::launch_dm_decay(a.data_ptr(), bf, a.stride(0), w2.data_ptr(), w0.data_ptr<float>(), (int)a.size(0), (int)a.size(1), (int)w2.size(0),
                       out.data_ptr<float>(), cur_stream(a));
  return out;
}

Tensor dm_wkv_scan(const Tensor& rkv, const Tensor& w, const Tensor& u, Tensor state, const Tensor& positions, const Tensor& qsl,
                   const Tensor& state_slots, const Tensor& counts, int64_t num_seqs, int64_t H, int64_t D) {
  const bool bf = act_bf16(rkv, "rkv");
  TORCH_CHECK(rkv.dim() == 3 && rkv.is_contiguous() && rkv.size(0) >= 3 && rkv.size(2) == H * D, "rkv must be [>=3, T, H*D]");
  const int64_t T = rkv.size(1), C = H * D;
  check_f32(w, "w", T * C);
  check_f32(u, "u", C);
  check_f32(state, "state");
  TORCH_CHECK(state.dim() == 4 && state.size(1) == H && state.size(2) == D && state.size(3) == D, "state must be [slots, H, D, D]");
  TORCH_CHECK(D >= 1 && D <= 128, "head size of the recurrence must be at most 128");
  check_step_meta(positions, qsl, state_slots, counts, T, num_seqs);
  Tensor out = at::zeros({T, C}, rkv.options().dtype(at::kFloat));
  dli::launch_dm_wkv_scan(rkv.data_ptr(), bf, T * C, w.data_ptr<float>(), u.data_ptr<float>(), state.data_ptr<float>(),
                          positions.data_ptr<int>(), qsl.data_ptr<int>(), state_slots.data_ptr<int>(), counts.data_ptr<int>(),
                          (int)num_seqs, (int)H, (int)D, out.data_ptr<float>(), cur_stream(rkv));
  return out;
}

Tensor dm_group_rms_gate(const Tensor& o, int64_t groups, const Tensor& w, double eps, const Tensor& gate, bool out_bf16) {
  check_f32(o, "o");
  TORCH_CHECK(o.dim() == 2 && groups >= 1 && o.size(1) % groups == 0, "o must be [T, groups * n]");
  const int64_t T = o.size(0), C = o.size(1);
  check_f32(w, "w", C);
  const bool gbf = act_bf16(gate, "gate");
  check_rows(gate, "gate");
  TORCH_CHECK(gate.size(0) == T && gate.size(1) == C, "gate must be [T, C]");
  Tensor out = at::empty({T, C}, o.options().dtype(out_bf16 ? at::kBFloat16 : at::kFloat));
  dli::launch_dm_group_rms_gate(o.data_ptr<float>(), (int)groups, w.data_ptr<float>(), (float)eps, gate.data_ptr(), gbf, gate.stride(0),
                                (int)T, (int)C, out.data_ptr(), out_bf16, cur_stream(o));
  return out;
}

std::tuple<Tensor, Tensor, Tensor> dm_sigmoid_route(const Tensor& h, const Tensor& router, int64_t E, int64_t K, double scale) {
  const bool bf = act_bf16(h, "h");
  check_rows(h, "h");
  const int64_t T = h.size(0), W = h.size(1);
  check_f32(router, "router");
  TORCH_CHECK(router.dim() == 2 && router.size(1) == W && (router.size(0) == E || router.size(0) == E + 1), "router must be [E (+1), W]");
  TORCH_CHECK(E >= 1 && E <= 64 && K >= 1 && K <= E, "at most 64 experts, 1 <= top <= experts");
  TORCH_CHECK(W * 4 <= kSmMaxLds, "row too wide");
  Tensor ids = at::empty({T, K}, h.options().dtype(at::kInt)), wts = at::empty({T, K}, h.options().dtype(at::kFloat));
  Tensor extra = at::empty({router.size(0) > E ? T : 0}, h.options().dtype(at::kFloat));
  dli::launch_dm_sigmoid_route(h.data_ptr(), bf, h.stride(0), router.data_ptr<float>(), (int)router.size(0), (int)E, (int)K, (float)scale,
                               (int)T, (int)W, ids.data_ptr<int>(), wts.data_ptr<float>(), extra.data_ptr<float>(), cur_stream(h));
  return {ids, wts, extra};
}

bool g_dm_grouped_experts = true;     // A/B knob (dm_set_grouped_experts): routed experts as grouped GEMMs on the matrix cores
void dm_set_grouped_experts(bool on) { g_dm_grouped_experts = on; }

// gated: `up` holds an expert's gate rows, then its up rows ([E, 2F, W]); the activation is silu(gate · h) ⊙ (up · h)
Tensor dm_relu2_experts(const Tensor& h, const Tensor& ids, const Tensor& wts, const Tensor& up, const Tensor& down, bool gated) {
  const bool bf = act_bf16(h, "h");
  check_rows(h, "h");
  const int64_t T = h.size(0), W = h.size(1);
  check_act_like(up, bf, "up");
  check_act_like(down, bf, "down");
  TORCH_CHECK(up.dim() == 3 && down.dim() == 3 && up.is_contiguous() && down.is_contiguous(), "expert weights must be contiguous 3-D");
  const int64_t E = up.size(0), F = gated ? up.size(1) / 2 : up.size(1);
  TORCH_CHECK(up.size(1) == (gated ? 2 * F : F) && up.size(2) == W && down.size(0) == E && down.size(1) == W && down.size(2) == F,
              "expert weights must be [E, F (gated: 2F), W] and [E, W, F]");
  check_i32(ids, "ids");
  check_f32(wts, "wts");
  TORCH_CHECK(ids.dim() == 2 && ids.size(0) == T && wts.dim() == 2 && wts.size(0) == T && wts.size(1) == ids.size(1), "ids / wts must be [T, K]");
  const int64_t K = ids.size(1);
  Tensor out = at::empty({T, W}, h.options());
  if (gated && bf && g_dm_grouped_experts && W % 128 == 0 && F % 64 == 0 && E <= 64 && (T * K >= 64 || F % 128 == 0) && h.is_contiguous() &&
      reinterpret_cast<uintptr_t>(h.data_ptr()) % 16 == 0) {
    // the expert kernels of the Mixtral path: weight streaming at decode size, else grouped GEMMs (gate / up tile pairs with
    // the silu product in the first epilogue)
    moe_apply(h, ids, wts, up, down, K, 0, E, 0, out, cur_stream(h));
    return out;
  }
  if (!gated && bf && g_dm_grouped_experts && W % 128 == 0 && F % 128 == 0 && E <= 64 && T * K >= 64 && h.stride(0) % 8 == 0 &&
      reinterpret_cast<uintptr_t>(h.data_ptr()) % 16 == 0) {
    // matrix-core path: the routed rows are bucketed by expert and both projections run as grouped GEMMs on 128-row tiles
    // (kernels/moe.hip: rows gathered by index, relu² in the first epilogue, gate weight and scatter in the second)
    auto stream = cur_stream(h);
    auto i32 = h.options().dtype(at::kInt);
    const int64_t n = T * K, TR = 128;
    const int64_t capacity = (n + TR - 1) / TR * TR + E * TR, max_tiles = capacity / TR;
    Tensor sorted = at::empty({capacity}, i32), tile_expert = at::empty({max_tiles}, i32), meta = at::empty({2}, i32);
    Tensor act = at::empty({capacity, F}, h.options());
    const int64_t col_blocks2 = W / TR, nk2 = F / 64;
    int64_t k_splits = 1;
    if (max_tiles * col_blocks2 < 1024)
      k_splits = std::min<int64_t>({(1024 + max_tiles * col_blocks2 - 1) / (max_tiles * col_blocks2), 16, nk2});
    const bool split = k_splits > 1;
    Tensor y = split ? at::empty({k_splits, n, W}, h.options().dtype(at::kFloat)) : at::empty({n, W}, h.options());
    dli::launch_moe_align(ids.data_ptr<int>(), (int)n, 0, (int)E, sorted.data_ptr<int>(), tile_expert.data_ptr<int>(),
                          meta.data_ptr<int>(), (int)capacity, (int)TR, stream);
    dli::launch_grouped_gemm(3, h.data_ptr(), h.stride(0), up.data_ptr(), F * W, sorted.data_ptr<int>(), tile_expert.data_ptr<int>(),
                             meta.data_ptr<int>(), wts.data_ptr<float>(), (int)K, act.data_ptr(), F, (int)W, (int)F, (int)max_tiles, 1, 0,
                             stream);
    dli::launch_grouped_gemm(split ? 2 : 1, act.data_ptr(), F, down.data_ptr(), W * F, sorted.data_ptr<int>(),
                             tile_expert.data_ptr<int>(), meta.data_ptr<int>(), wts.data_ptr<float>(), (int)K, y.data_ptr(), W, (int)F,
                             (int)W, (int)max_tiles, (int)k_splits, n * W, stream);
    dli::launch_moe_sum(y.data_ptr(), split, (int)k_splits, n * W, ids.data_ptr<int>(), 0, (int)E, (int)K, (int)T, (int)W, out.data_ptr(),
                        stream);
    return out;
  }
  TORCH_CHECK(W * 4 <= kSmMaxLds && K * F * 4 <= kSmMaxLds, "rows too wide");
  Tensor act = at::empty({T * K, F}, h.options());
  dli::launch_dm_experts(h.data_ptr(), bf, h.stride(0), ids.data_ptr<int>(), wts.data_ptr<float>(), (int)K, up.data_ptr(), down.data_ptr(),
                         (int)T, (int)F, (int)W, act.data_ptr(), out.data_ptr(), gated ? 1 : 0, (int)E, 0.f, cur_stream(h));
  return out;
}

Tensor dm_relu2_rows(const Tensor& x) {
  const bool bf = act_bf16(x, "x");
  check_rows(x, "x");
  Tensor out = at::empty({x.size(0), x.size(1)}, x.options());
  dli::launch_dm_relu2_rows(x.data_ptr(), bf, x.stride(0), (int)x.size(0), (int)x.size(1), out.data_ptr(), cur_stream(x));
  return out;
}

void dm_gated_combine(Tensor x, double mult, const Tensor& p0, const Tensor& p1, double s0, double s1, const Tensor& g1, const Tensor& b1,
                      const c10::optional<Tensor>& ff, const c10::optional<Tensor>& shared, const c10::optional<Tensor>& sg,
                      const c10::optional<Tensor>& g2, const c10::optional<Tensor>& b2) {
  check_f32(x, "x");
  TORCH_CHECK(x.dim() == 2, "x must be [T, W]");
  const int64_t T = x.size(0), W = x.size(1);
  const bool bf = act_bf16(p0, "p0");
  auto full = [&](const Tensor& t, const char* name) {
    check_act_like(t, bf, name);
    TORCH_CHECK(t.dim() == 2 && t.is_contiguous() && t.size(0) == T && t.size(1) == W, name, " must be contiguous [T, W]");
    return t.data_ptr();
  };
  auto view = [&](const Tensor& t, const char* name) {
    check_act_like(t, bf, name);
    check_rows(t, name);
    TORCH_CHECK(t.size(0) == T && t.size(1) == W, name, " must be [T, W]");
    return t.data_ptr();
  };
  const void* p0p = full(p0, "p0");
  const void* p1p = full(p1, "p1");
  const void* g1p = view(g1, "g1");
  check_f32(b1, "b1", W);
  TORCH_CHECK(g2.has_value() == b2.has_value(), "g2 and b2 come together");
  TORCH_CHECK(g2.has_value() || !(ff.has_value() || shared.has_value()), "a feed-forward term needs its gate");
  const void* ffp = ff.has_value() ? full(*ff, "ff") : nullptr;
  const void* shp = shared.has_value() ? full(*shared, "shared") : nullptr;
  const float* sgp = opt_f32(sg, "sg", T);
  const void* g2p = g2.has_value() ? view(*g2, "g2") : nullptr;
  const float* b2p = opt_f32(b2, "b2", W);
  dli::launch_dm_gated_combine(x.data_ptr<float>(), (float)mult, p0p, p1p, (float)s0, (float)s1, g1p, g1.stride(0), b1.data_ptr<float>(), ffp,
                               shp, sgp, g2p, g2.has_value() ? g2->stride(0) : 0, b2p, bf, (int)T, (int)W, cur_stream(x));
}
