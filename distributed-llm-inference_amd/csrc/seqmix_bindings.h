// torch.ops.dli.sm_* — argument checks around the launchers of kernels/seqmix.hip (heterogeneous decoder stacks).
// Included by torch_bindings.cpp inside its anonymous namespace (uses its Tensor alias, cur_stream and check_i32).
// Every shape the kernels index with is checked here: the kernels themselves do no bounds checks.
#pragma once

bool act_bf16(const Tensor& t, const char* name) {
  TORCH_CHECK(t.is_cuda(), name, " must be a GPU tensor");
  TORCH_CHECK(t.scalar_type() == at::kBFloat16 || t.scalar_type() == at::kFloat, name, " must be bfloat16 or float32");
  return t.scalar_type() == at::kBFloat16;
}
void check_f32(const Tensor& t, const char* name, int64_t numel = -1) {
  TORCH_CHECK(t.is_cuda() && t.scalar_type() == at::kFloat && t.is_contiguous(), name, " must be a contiguous float32 GPU tensor");
  TORCH_CHECK(numel < 0 || t.numel() == numel, name, " has ", t.numel(), " elements, expected ", numel);
}
void check_rows(const Tensor& t, const char* name) {
  TORCH_CHECK(t.dim() == 2 && t.stride(1) == 1, name, " must be 2-D with contiguous rows");
}
const float* opt_f32(const c10::optional<Tensor>& t, const char* name, int64_t numel) {
  if (!t.has_value()) return nullptr;
  check_f32(*t, name, numel);
  return t->data_ptr<float>();
}
constexpr int64_t kSmMaxLds = 60 * 1024;     // dynamic LDS a kernel may ask for without opting in to more
constexpr int64_t kSmPageTokens = 32;        // tokens per cache page (config.KV_BLOCK_SIZE, kernels/common.h kBlockTokens)

Tensor sm_layer_norm(const Tensor& x, const Tensor& w, const Tensor& b, double eps, bool out_bf16) {
  check_f32(x, "x");
  TORCH_CHECK(x.dim() == 2, "x must be [rows, W]");
  const int64_t W = x.size(1);
  check_f32(w, "w", W);
  check_f32(b, "b", W);
  TORCH_CHECK(W * 4 <= kSmMaxLds, "row too wide");
  Tensor out = at::empty({x.size(0), W}, x.options().dtype(out_bf16 ? at::kBFloat16 : at::kFloat));
  dli::launch_sm_layer_norm(x.data_ptr<float>(), w.data_ptr<float>(), b.data_ptr<float>(), (float)eps, (int)x.size(0), (int)W,
                            out.data_ptr(), out_bf16, cur_stream(x));
  return out;
}

std::tuple<Tensor, Tensor> sm_ln_shift(const Tensor& x, const c10::optional<Tensor>& add, const Tensor& w, const Tensor& b, double eps,
                                       const Tensor& mix, Tensor state, const Tensor& positions, const Tensor& token_seq,
                                       const Tensor& qsl, const Tensor& state_slots, const Tensor& counts, int64_t num_seqs,
                                       bool out_bf16) {
  check_f32(x, "x");
  TORCH_CHECK(x.dim() == 2, "x must be [T, W]");
  const int64_t T = x.size(0), W = x.size(1);
  check_f32(w, "w", W);
  check_f32(b, "b", W);
  check_f32(mix, "mix", W);
  check_f32(state, "state");
  TORCH_CHECK(state.dim() == 2 && state.size(1) == W, "state must be [slots, W]");
  check_i32(positions, "positions");
  check_i32(token_seq, "token_seq");
  check_i32(qsl, "query_start_loc");
  check_i32(state_slots, "state_slots");
  check_i32(counts, "counts");
  TORCH_CHECK(positions.numel() >= T && token_seq.numel() >= T && counts.numel() >= 4, "step metadata shorter than the batch");
  TORCH_CHECK(num_seqs >= 0 && qsl.numel() >= num_seqs + 1 && state_slots.numel() >= num_seqs, "batch-row metadata too short");
  TORCH_CHECK(2 * W * 4 <= kSmMaxLds, "row too wide");
  Tensor xout = x;
  const float* addp = nullptr;
  if (add.has_value()) {
    check_f32(*add, "add", T * W);
    addp = add->data_ptr<float>();
    xout = at::empty_like(x);
  }
  Tensor out = at::empty({T, W}, x.options().dtype(out_bf16 ? at::kBFloat16 : at::kFloat));
  dli::launch_sm_ln_shift(x.data_ptr<float>(), addp, addp ? xout.data_ptr<float>() : nullptr, w.data_ptr<float>(), b.data_ptr<float>(),
                          mix.data_ptr<float>(), state.data_ptr<float>(), positions.data_ptr<int>(), token_seq.data_ptr<int>(),
                          qsl.data_ptr<int>(), state_slots.data_ptr<int>(), counts.data_ptr<int>(), (int)T, (int)num_seqs, (float)eps,
                          (int)W, out.data_ptr(), out_bf16, cur_stream(x));
  return {out, xout};
}

Tensor sm_add_ln(Tensor x, const Tensor& y, const Tensor& w, const Tensor& b, double eps, double mult, const c10::optional<Tensor>& w2,
                 const c10::optional<Tensor>& b2, bool out_bf16) {
  check_f32(x, "x");
  TORCH_CHECK(x.dim() == 2, "x must be [T, W]");
  const int64_t T = x.size(0), W = x.size(1);
  const bool ybf = act_bf16(y, "y");
  check_rows(y, "y");
  TORCH_CHECK(y.size(0) == T && y.size(1) == W, "y must be shaped like x");
  check_f32(w, "w", W);
  check_f32(b, "b", W);
  TORCH_CHECK(w2.has_value() == b2.has_value(), "w2 and b2 come together");
  TORCH_CHECK(W * 4 <= kSmMaxLds, "row too wide");
  const float* w2p = opt_f32(w2, "w2", W);
  const float* b2p = opt_f32(b2, "b2", W);
  Tensor out = at::empty({w2p ? T : 0, W}, x.options().dtype(out_bf16 ? at::kBFloat16 : at::kFloat));
  dli::launch_sm_add_ln(x.data_ptr<float>(), y.data_ptr(), ybf, y.stride(0), w.data_ptr<float>(), b.data_ptr<float>(), (float)mult, w2p,
                        b2p, (float)eps, (int)T, (int)W, out.data_ptr(), out_bf16, cur_stream(x));
  return out;
}

Tensor sm_rms_gate(const Tensor& o, const c10::optional<Tensor>& w, double eps, const Tensor& gate, bool out_bf16, int64_t groups,
                   bool silu) {
  check_f32(o, "o");
  TORCH_CHECK(o.dim() == 2 || o.dim() == 3, "o must be [T, N] or planes of partial sums [parts, T, N]");
  const int64_t parts = o.dim() == 3 ? o.size(0) : 1;
  const int64_t T = o.size(-2), N = o.size(-1);
  TORCH_CHECK(N * 4 <= kSmMaxLds, "row too wide");
  const float* wp = opt_f32(w, "w", N);
  TORCH_CHECK(groups >= 1 && N % groups == 0, "the row does not divide into that many groups");
  const bool gbf = act_bf16(gate, "gate");
  check_rows(gate, "gate");
  TORCH_CHECK(gate.size(0) == T && gate.size(1) == N, "gate must be [T, N]");
  Tensor out = at::empty({T, N}, o.options().dtype(out_bf16 ? at::kBFloat16 : at::kFloat));
  dli::launch_sm_rms_gate(o.data_ptr<float>(), (int)parts, wp, (float)eps, gate.data_ptr(), gbf, gate.stride(0), (int)T, (int)N,
                          out.data_ptr(), out_bf16, (int)groups, silu, cur_stream(o));
  return out;
}

Tensor sm_relu2(const Tensor& x) {
  const bool bf = act_bf16(x, "x");
  TORCH_CHECK(x.is_contiguous(), "x must be contiguous");
  Tensor out = at::empty_like(x);
  dli::launch_sm_relu2(x.data_ptr(), out.data_ptr(), x.numel(), bf, cur_stream(x));
  return out;
}

Tensor sm_softcap(const Tensor& x, double cap) {
  const bool bf = act_bf16(x, "x");
  TORCH_CHECK(x.is_contiguous() && cap > 0, "x must be contiguous and cap positive");
  Tensor out = at::empty(x.sizes(), x.options().dtype(at::kFloat));
  dli::launch_sm_softcap(x.data_ptr(), bf, out.data_ptr<float>(), (float)cap, x.numel(), cur_stream(x));
  return out;
}

void sm_qk_norm_cache(Tensor qkv, const Tensor& qw, const Tensor& kw, double eps, const Tensor& slot_mapping, Tensor k_cache,
                      Tensor v_cache, int64_t H, int64_t G, int64_t D, int64_t Dv) {
  const bool bf = act_bf16(qkv, "qkv");
  check_rows(qkv, "qkv");
  const int64_t T = qkv.size(0);
  TORCH_CHECK(H > 0 && G > 0 && H % G == 0 && qkv.size(1) == (H + G) * D + G * Dv, "qkv row does not match the head sizes");
  check_f32(qw, "qw", D);
  check_f32(kw, "kw", D);
  check_i32(slot_mapping, "slot_mapping");
  TORCH_CHECK(slot_mapping.numel() >= T, "slot_mapping shorter than the batch");
  TORCH_CHECK(k_cache.is_cuda() && k_cache.is_contiguous() && k_cache.scalar_type() == qkv.scalar_type() && k_cache.size(-1) == G * D,
              "k_cache must be contiguous [..., G*D] of the activation type");
  TORCH_CHECK(v_cache.is_cuda() && v_cache.is_contiguous() && v_cache.scalar_type() == qkv.scalar_type() && v_cache.size(-1) == G * Dv &&
                  v_cache.numel() / (G * Dv) == k_cache.numel() / (G * D),
              "v_cache must be contiguous [..., G*Dv] with as many rows as k_cache");
  dli::launch_sm_qk_norm_cache(qkv.data_ptr(), bf, qkv.stride(0), qw.data_ptr<float>(), kw.data_ptr<float>(), (float)eps,
                               slot_mapping.data_ptr<int>(), k_cache.data_ptr(), v_cache.data_ptr(), (int)T, (int)H, (int)G, (int)D,
                               (int)Dv, cur_stream(qkv));
}

void sm_latent_prep(Tensor q, const Tensor& dkv, const Tensor& cw, double eps, const Tensor& positions, const Tensor& inv_freq,
                    int64_t rot_dims, const Tensor& slot_mapping, Tensor cache, int64_t H, int64_t D, int64_t R, int64_t C) {
  const bool bf = act_bf16(q, "q");
  check_rows(q, "q");
  check_rows(dkv, "dkv");
  const int64_t T = q.size(0);
  TORCH_CHECK(dkv.scalar_type() == q.scalar_type() && dkv.is_cuda() && dkv.size(0) == T, "dkv must match q");
  TORCH_CHECK(q.size(1) == H * (D + R) && dkv.size(1) == C + R, "q / dkv rows do not match the head sizes");
  TORCH_CHECK(rot_dims >= 0 && rot_dims % 2 == 0 && rot_dims <= R, "rot_dims must be even and at most R");
  check_f32(cw, "cw", C);
  TORCH_CHECK(inv_freq.is_cuda() && inv_freq.scalar_type() == at::kDouble && inv_freq.is_contiguous() && inv_freq.numel() == rot_dims / 2,
              "inv_freq must be float64 [rot_dims / 2]");
  check_i32(positions, "positions");
  check_i32(slot_mapping, "slot_mapping");
  TORCH_CHECK(positions.numel() >= T && slot_mapping.numel() >= T, "step metadata shorter than the batch");
  TORCH_CHECK(cache.is_cuda() && cache.is_contiguous() && cache.scalar_type() == q.scalar_type() && cache.size(-1) == C + R,
              "cache must be contiguous [..., C+R] of the activation type");
  dli::launch_sm_latent_prep(q.data_ptr(), bf, q.stride(0), dkv.data_ptr(), dkv.stride(0), cw.data_ptr<float>(), (float)eps,
                             positions.data_ptr<int>(), inv_freq.data_ptr<double>(), (int)rot_dims, slot_mapping.data_ptr<int>(),
                             cache.data_ptr(), (int)T, (int)H, (int)D, (int)R, (int)C, cur_stream(q));
}

// per-head output gate of the attention kernels: [T, H] rows (pre-activation, row-strided view) of the queries' dtype
const void* head_gate(const c10::optional<Tensor>& gate, const Tensor& q1, int64_t T, int64_t H, int64_t* stride) {
  *stride = 0;
  if (!gate.has_value()) return nullptr;
  TORCH_CHECK(gate->is_cuda() && gate->scalar_type() == q1.scalar_type() && gate->dim() == 2 && gate->stride(1) == 1 &&
                  gate->size(0) == T && gate->size(1) == H, "gate must be [T, H] like the queries");
  *stride = gate->stride(0);
  return gate->data_ptr();
}

void sm_token_attention(Tensor out, const Tensor& q1, const c10::optional<Tensor>& q2, const Tensor& k_cache,
                        const c10::optional<Tensor>& v_cache, const Tensor& block_tables, const Tensor& positions,
                        const Tensor& token_seq, int64_t G, int64_t Dv, double scale, int64_t window, const c10::optional<Tensor>& temp,
                        const c10::optional<Tensor>& r1, const c10::optional<Tensor>& r2, int64_t rows,
                        const c10::optional<Tensor>& gate, const c10::optional<Tensor>& sink) {
  const bool bf = act_bf16(q1, "q1");
  TORCH_CHECK(q1.dim() == 3 && q1.stride(2) == 1, "q1 must be [T, H, D1] with a contiguous last dim");
  TORCH_CHECK(rows < 0 || rows <= q1.size(0), "rows past the batch");
  const int64_t T = q1.size(0), H = q1.size(1), D1 = q1.size(2);
  int64_t D2 = 0;
  if (q2.has_value()) {
    TORCH_CHECK(q2->is_cuda() && q2->scalar_type() == q1.scalar_type() && q2->dim() == 3 && q2->stride(2) == 1 && q2->size(0) == T &&
                    q2->size(1) == H, "q2 must be [T, H, D2] like q1");
    D2 = q2->size(2);
  }
  TORCH_CHECK(G > 0 && H % G == 0, "query heads must be a multiple of the key heads");
  const int64_t Dk = D1 + D2;
  TORCH_CHECK(k_cache.is_cuda() && k_cache.is_contiguous() && k_cache.scalar_type() == q1.scalar_type() && k_cache.dim() == 3 &&
                  k_cache.size(1) == kSmPageTokens && k_cache.size(2) == G * Dk, "k_cache must be [pages, 32, G*(D1+D2)]");
  const Tensor& vc = v_cache.has_value() ? *v_cache : k_cache;
  int64_t vhead = Dk;
  if (v_cache.has_value()) {
    TORCH_CHECK(vc.is_cuda() && vc.is_contiguous() && vc.scalar_type() == q1.scalar_type() && vc.dim() == 3 && vc.size(0) == k_cache.size(0) &&
                    vc.size(1) == kSmPageTokens && vc.size(2) == G * Dv, "v_cache must be [pages, 32, G*Dv]");
    vhead = Dv;
  } else {
    TORCH_CHECK(Dv <= Dk, "values read from the key rows cannot be wider than a key");
  }
  TORCH_CHECK(Dv > 0 && Dv <= 8192, "value size must be in 1..8192");
  TORCH_CHECK(out.is_cuda() && out.scalar_type() == q1.scalar_type() && out.dim() == 3 && out.stride(2) == 1 && out.size(0) == T &&
                  out.size(1) == H && out.size(2) == Dv, "out must be [T, H, Dv]");
  check_i32(block_tables, "block_tables");
  check_i32(positions, "positions");
  check_i32(token_seq, "token_seq");
  TORCH_CHECK(block_tables.dim() == 2 && positions.numel() >= T && token_seq.numel() >= T, "step metadata shorter than the batch");
  TORCH_CHECK(r1.has_value() == r2.has_value(), "r1 and r2 come together");
  TORCH_CHECK((Dk + 4 * std::min<int64_t>(Dv, 512) + 8) * 4 <= kSmMaxLds, "head sizes exceed the kernel's LDS budget");
  int64_t g_ts = 0;
  const void* gp = head_gate(gate, q1, T, H, &g_ts);
  // few rows (decode steps): long key ranges are cut over several workgroups, partial results in `part`
  const int64_t n_rows = rows < 0 ? T : rows;
  const int nsplit = Dv > 512 ? 1 : dli::sm_token_attention_splits((int)n_rows, (int)H, (int)G);
  Tensor part;
  if (nsplit > 1) part = at::empty({n_rows, H, nsplit, Dv + 2}, q1.options().dtype(at::kFloat));
  dli::launch_sm_token_attention(out.data_ptr(), out.stride(0), out.stride(1), q1.data_ptr(), q1.stride(0), q1.stride(1), (int)D1,
                                 q2.has_value() ? q2->data_ptr() : nullptr, q2.has_value() ? q2->stride(0) : 0,
                                 q2.has_value() ? q2->stride(1) : 0, (int)D2, k_cache.data_ptr(), (int)(G * Dk), vc.data_ptr(),
                                 (int)vc.size(2), (int)vhead, (int)Dv, block_tables.data_ptr<int>(), (int)block_tables.size(1),
                                 positions.data_ptr<int>(), token_seq.data_ptr<int>(), (int)n_rows, (int)H, (int)G, (float)scale,
                                 (int)window, opt_f32(temp, "temp", H), opt_f32(r1, "r1", H), opt_f32(r2, "r2", H), bf, nsplit,
                                 nsplit > 1 ? part.data_ptr<float>() : nullptr, gp, g_ts, opt_f32(sink, "sink", H), cur_stream(q1));
}

// Decode rows (the first `rows` tokens) of a mixer whose heads share key / value heads in groups of 8 or more, heads as the
// MFMA columns; bf16 only.  False: shapes that kernel does not take — nothing was launched.
bool sm_head_decode_attention(Tensor out, const Tensor& q1, const c10::optional<Tensor>& q2, const Tensor& k_cache,
                              const c10::optional<Tensor>& v_cache, const Tensor& block_tables, const Tensor& positions,
                              const Tensor& token_seq, int64_t G, int64_t Dv, double scale, int64_t window,
                              const c10::optional<Tensor>& temp, const c10::optional<Tensor>& r1, const c10::optional<Tensor>& r2,
                              int64_t rows, const c10::optional<Tensor>& gate, const c10::optional<Tensor>& sink) {
  TORCH_CHECK(q1.is_cuda() && q1.scalar_type() == at::kBFloat16 && q1.dim() == 3 && q1.stride(2) == 1, "q1 must be bfloat16 [T, H, D1]");
  const int64_t T = q1.size(0), H = q1.size(1), D1 = q1.size(2);
  TORCH_CHECK(rows >= 0 && rows <= T, "rows past the batch");
  int64_t D2 = 0;
  if (q2.has_value()) {
    TORCH_CHECK(q2->is_cuda() && q2->scalar_type() == at::kBFloat16 && q2->dim() == 3 && q2->stride(2) == 1 && q2->size(0) == T &&
                    q2->size(1) == H, "q2 must be [T, H, D2] like q1");
    D2 = q2->size(2);
  }
  TORCH_CHECK(G > 0 && H % G == 0, "query heads must be a multiple of the key heads");
  const int64_t Dk = D1 + D2;
  TORCH_CHECK(k_cache.is_cuda() && k_cache.is_contiguous() && k_cache.scalar_type() == at::kBFloat16 && k_cache.dim() == 3 &&
                  k_cache.size(1) == kSmPageTokens && k_cache.size(2) == G * Dk, "k_cache must be [pages, 32, G*(D1+D2)]");
  const Tensor& vc = v_cache.has_value() ? *v_cache : k_cache;
  int64_t vhead = Dk;
  if (v_cache.has_value()) {
    TORCH_CHECK(vc.is_cuda() && vc.is_contiguous() && vc.scalar_type() == at::kBFloat16 && vc.dim() == 3 && vc.size(0) == k_cache.size(0) &&
                    vc.size(1) == kSmPageTokens && vc.size(2) == G * Dv, "v_cache must be [pages, 32, G*Dv]");
    vhead = Dv;
  } else {
    TORCH_CHECK(Dv <= Dk, "values read from the key rows cannot be wider than a key");
  }
  TORCH_CHECK(out.is_cuda() && out.scalar_type() == at::kBFloat16 && out.dim() == 3 && out.stride(2) == 1 && out.size(0) == T &&
                  out.size(1) == H && out.size(2) == Dv, "out must be [T, H, Dv]");
  check_i32(block_tables, "block_tables");
  check_i32(positions, "positions");
  check_i32(token_seq, "token_seq");
  TORCH_CHECK(block_tables.dim() == 2 && positions.numel() >= T && token_seq.numel() >= T, "step metadata shorter than the batch");
  TORCH_CHECK(r1.has_value() == r2.has_value(), "r1 and r2 come together");
  int64_t g_ts = 0;
  const void* gp = head_gate(gate, q1, T, H, &g_ts);
  const int nsplit = dli::sm_head_decode_splits((int)rows, (int)H, (int)G);
  Tensor part;
  if (nsplit > 1) part = at::empty({std::max<int64_t>(rows, 1), H, nsplit, Dv + 2}, q1.options().dtype(at::kFloat));
  return dli::launch_sm_head_decode_attention(out.data_ptr(), out.stride(0), out.stride(1), q1.data_ptr(), q1.stride(0), q1.stride(1),
                                              (int)D1, q2.has_value() ? q2->data_ptr() : nullptr, q2.has_value() ? q2->stride(0) : 0,
                                              q2.has_value() ? q2->stride(1) : 0, (int)D2, k_cache.data_ptr(), (int)(G * Dk),
                                              vc.data_ptr(), (int)vc.size(2), (int)vhead, (int)Dv, block_tables.data_ptr<int>(),
                                              (int)block_tables.size(1), positions.data_ptr<int>(), token_seq.data_ptr<int>(), (int)rows,
                                              (int)H, (int)G, (float)scale, (int)window, opt_f32(temp, "temp", H), opt_f32(r1, "r1", H),
                                              opt_f32(r2, "r2", H), nsplit, nsplit > 1 ? part.data_ptr<float>() : nullptr, gp, g_ts, opt_f32(sink, "sink", H),
                                              cur_stream(q1));
}

// Prefill tiles (64 queries of one sequence's chunk each) on the matrix cores; bf16 only.  False: shapes the tile kernel does
// not take — nothing was launched, the caller uses the per-token kernel.
bool sm_tile_attention(Tensor out, const Tensor& q1, const c10::optional<Tensor>& q2, const Tensor& k_cache,
                       const c10::optional<Tensor>& v_cache, const Tensor& block_tables, const Tensor& seq_lens, const Tensor& qsl,
                       const Tensor& tile_seq, const Tensor& tile_q0, int64_t num_tiles, const c10::optional<Tensor>& counts, int64_t G,
                       int64_t Dv, double scale, int64_t window, const c10::optional<Tensor>& temp, const c10::optional<Tensor>& r1,
                       const c10::optional<Tensor>& r2, const c10::optional<Tensor>& gate, const c10::optional<Tensor>& sink) {
  TORCH_CHECK(q1.is_cuda() && q1.scalar_type() == at::kBFloat16 && q1.dim() == 3 && q1.stride(2) == 1, "q1 must be bfloat16 [T, H, D1]");
  const int64_t T = q1.size(0), H = q1.size(1), D1 = q1.size(2);
  int64_t D2 = 0;
  if (q2.has_value()) {
    TORCH_CHECK(q2->is_cuda() && q2->scalar_type() == at::kBFloat16 && q2->dim() == 3 && q2->stride(2) == 1 && q2->size(0) == T &&
                    q2->size(1) == H, "q2 must be [T, H, D2] like q1");
    D2 = q2->size(2);
  }
  TORCH_CHECK(G > 0 && H % G == 0, "query heads must be a multiple of the key heads");
  const int64_t Dk = D1 + D2;
  TORCH_CHECK(k_cache.is_cuda() && k_cache.is_contiguous() && k_cache.scalar_type() == at::kBFloat16 && k_cache.dim() == 3 &&
                  k_cache.size(1) == kSmPageTokens && k_cache.size(2) == G * Dk, "k_cache must be [pages, 32, G*(D1+D2)]");
  const Tensor& vc = v_cache.has_value() ? *v_cache : k_cache;
  int64_t vhead = Dk;
  if (v_cache.has_value()) {
    TORCH_CHECK(vc.is_cuda() && vc.is_contiguous() && vc.scalar_type() == at::kBFloat16 && vc.dim() == 3 && vc.size(0) == k_cache.size(0) &&
                    vc.size(1) == kSmPageTokens && vc.size(2) == G * Dv, "v_cache must be [pages, 32, G*Dv]");
    vhead = Dv;
  } else {
    TORCH_CHECK(Dv <= Dk, "values read from the key rows cannot be wider than a key");
  }
  TORCH_CHECK(out.is_cuda() && out.scalar_type() == at::kBFloat16 && out.dim() == 3 && out.stride(2) == 1 && out.size(0) == T &&
                  out.size(1) == H && out.size(2) == Dv, "out must be [T, H, Dv]");
  check_i32(block_tables, "block_tables");
  check_i32(seq_lens, "seq_lens");
  check_i32(qsl, "query_start_loc");
  check_i32(tile_seq, "tile_seq");
  check_i32(tile_q0, "tile_q0");
  TORCH_CHECK(block_tables.dim() == 2 && num_tiles >= 0 && tile_seq.numel() >= num_tiles && tile_q0.numel() >= num_tiles,
              "tile list shorter than the launch");
  const int* cnt = nullptr;
  if (counts.has_value()) {
    check_i32(*counts, "counts");
    TORCH_CHECK(counts->numel() >= 4, "counts must hold 4 values");
    cnt = counts->data_ptr<int>();
  }
  TORCH_CHECK(r1.has_value() == r2.has_value(), "r1 and r2 come together");
  int64_t g_ts = 0;
  const void* gp = head_gate(gate, q1, T, H, &g_ts);
  return dli::launch_sm_tile_attention(out.data_ptr(), out.stride(0), out.stride(1), q1.data_ptr(), q1.stride(0), q1.stride(1), (int)D1,
                                       q2.has_value() ? q2->data_ptr() : nullptr, q2.has_value() ? q2->stride(0) : 0,
                                       q2.has_value() ? q2->stride(1) : 0, (int)D2, k_cache.data_ptr(), (int)(G * Dk), vc.data_ptr(),
                                       (int)vc.size(2), (int)vhead, (int)Dv, block_tables.data_ptr<int>(), (int)block_tables.size(1),
                                       seq_lens.data_ptr<int>(), qsl.data_ptr<int>(), tile_seq.data_ptr<int>(), tile_q0.data_ptr<int>(),
                                       (int)num_tiles, cnt, (int)H, (int)G, (float)scale, (int)window, opt_f32(temp, "temp", H),
                                       opt_f32(r1, "r1", H), opt_f32(r2, "r2", H), gp, g_ts, opt_f32(sink, "sink", H), cur_stream(q1));
}

Tensor sm_lightning_scan(const Tensor& qkvg, Tensor state, const Tensor& positions, const Tensor& qsl, const Tensor& state_slots,
                         const Tensor& counts, int64_t num_seqs, int64_t H, int64_t D, int64_t Dv, const Tensor& decay,
                         const c10::optional<Tensor>& tile_seq, const c10::optional<Tensor>& tile_q0, int64_t num_tiles,
                         bool plain_act) {
  const bool bf = act_bf16(qkvg, "qkvg");
  check_rows(qkvg, "qkvg");
  const int64_t T = qkvg.size(0);
  TORCH_CHECK(qkvg.size(1) >= 2 * H * D + H * Dv, "qkvg row narrower than q | k | v");
  TORCH_CHECK(D > 0 && D <= 1024, "key size must be in 1..1024");     // a wave keeps at most 256 state rows, D is cut in up to 4 parts
  check_f32(state, "state");
  TORCH_CHECK(state.dim() == 4 && state.size(1) == H && state.size(2) == D && state.size(3) == Dv, "state must be [slots, H, D, Dv]");
  check_f32(decay, "decay", H);
  check_i32(positions, "positions");
  check_i32(qsl, "query_start_loc");
  check_i32(state_slots, "state_slots");
  check_i32(counts, "counts");
  TORCH_CHECK(positions.numel() >= T && counts.numel() >= 4 && num_seqs >= 0 && qsl.numel() >= num_seqs + 1 &&
                  state_slots.numel() >= num_seqs, "step metadata shorter than the batch");
  // one plane of partial outputs per part of the state rows (summed by sm_rms_gate)
  const int64_t parts = dli::sm_lightning_parts((int)D);
  Tensor out = at::zeros({parts, T, H * Dv}, qkvg.options().dtype(at::kFloat));
  // block path of prefill chunks: 64-token blocks = the step's prefill tiles; one [H, D, Dv] workspace row per block
  const int* ts = nullptr;
  const int* tq = nullptr;
  Tensor ws;
  if (num_tiles > 0) {
    TORCH_CHECK(tile_seq.has_value() && tile_q0.has_value(), "a block list needs tile_seq and tile_q0");
    check_i32(*tile_seq, "tile_seq");
    check_i32(*tile_q0, "tile_q0");
    TORCH_CHECK(tile_seq->numel() >= num_tiles && tile_q0->numel() >= num_tiles, "tile list shorter than the launch");
    ts = tile_seq->data_ptr<int>();
    tq = tile_q0->data_ptr<int>();
    ws = at::empty({T / 64 + num_seqs + 2, H, D, Dv}, state.options());
  }
  dli::launch_sm_lightning_scan(qkvg.data_ptr(), bf, qkvg.stride(0), state.data_ptr<float>(), positions.data_ptr<int>(),
                                qsl.data_ptr<int>(), state_slots.data_ptr<int>(), counts.data_ptr<int>(), (int)num_seqs, (int)H, (int)D,
                                (int)Dv, decay.data_ptr<float>(), out.data_ptr<float>(), T * H * Dv, ts, tq, (int)num_tiles,
                                num_tiles > 0 ? ws.data_ptr<float>() : nullptr, plain_act, cur_stream(qkvg));
  return out;
}
