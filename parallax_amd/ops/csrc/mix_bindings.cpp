// Python bindings of the sequence-mixer kernels (extension parallax_amd.ops._mix):
// fp32-residual layer norm, sliding-window latent attention, gated linear
// attention, sandwich RMS norm with depth averaging, row-cache attention
// (differential / pooled sliding window), xIELU. Every entry point checks shapes and types on the host before a
// launch; activation tensors are bf16 or float32 (one template instance each).

#include <ATen/hip/HIPContext.h>
#include <torch/extension.h>

#include <hip/hip_runtime.h>

#include <algorithm>

extern "C" {
void launch_add_layernorm(float*, const void*, int64_t, int, const void*, float,
                          const void*, const void*, float, void*, int, int, int,
                          hipStream_t);
void launch_latent_kv_store(const void*, int64_t, const void*, float,
                            const float*, float, int, const int*,
                            const int64_t*, void*, int, int, int, int,
                            hipStream_t);
void launch_rope_rows(float*, const void*, int64_t, int64_t, int, const float*,
                      float, int, const int*, int, int, int, int, hipStream_t);
void launch_latent_window_attention(float*, float*, const float*, const float*,
                                    const void*, const int*, int, const int*,
                                    const int*, int, int, int, int, int, int,
                                    float, int, int, hipStream_t);
void launch_gla_recurrence(float*, const void*, const void*, const void*,
                           const void*, int64_t, int64_t, int64_t, int64_t,
                           const void*, float*, const int64_t*, const int*,
                           const int*, int, int, int, int, float, float, int,
                           hipStream_t);
void launch_gated_rmsnorm(void*, const float*, const void*, int64_t,
                          const void*, float, int, int, int, int, hipStream_t);
void launch_sandwich_rmsnorm(float*, const void*, int64_t, int, const void*,
                             float*, int64_t, int, const float*, const void*,
                             float, float, void*, const void*, const int*, int,
                             int, int, hipStream_t);
void launch_xielu(void*, const void*, int64_t, float, float, int, hipStream_t);
void launch_qkv_store(float*, const void*, int64_t, const void*, int64_t,
                      const void*, int64_t, const int*, const int64_t*, void*,
                      int, int, int, int, float, float, int, const float*,
                      const float*, const float*, float, int, int, int,
                      const float*, int, float*, int, int, hipStream_t);
void launch_pool_cache_update(const void*, float*, const int*, int, const int*,
                              const int*, const int64_t*, int, int, int, int,
                              int, int, hipStream_t);
int row_attention_heads_per_group(int);
int row_attention_prefill_supported(int, int);
int row_attention_prefill_rotates(int, int);
void launch_rotate_heads_table(void*, const float*, const float*, int, int,
                               int, float, int, int, hipStream_t);
void launch_row_attention_prefill(void*, float*, const float*, const void*,
                                  const float*, const int*, int, const int*,
                                  int, const int*, int, int, int, int, int, int,
                                  int, int, int, int, float, float, float,
                                  float, float, const float*, const void*,
                                  int64_t, int, const float*, int, int,
                                  hipStream_t);
void launch_row_attention(void*, float*, float*, const float*, const void*,
                          const float*, const int*, int, const int*, const int*,
                          int, int, int, int, int, int, int, int, int, int,
                          float, float, float, float, float, int, const float*,
                          const void*, int64_t, int, const float*, int, int,
                          hipStream_t);
void launch_group_rmsnorm_add(float*, const void*, int64_t, const void*,
                              int64_t, const void*, float, void*, int, int,
                              int, int, hipStream_t);
void launch_pair_hash_embedding(float*, const int64_t*, const int64_t*,
                                const void*, const void*, float, int64_t,
                                int64_t, int64_t, int64_t, int, int, int,
                                hipStream_t);
void launch_relu_squared(void*, const void*, int64_t, int, int, int,
                         hipStream_t);
void launch_rotate_heads(void*, const float*, const float*, const int*, int,
                         int, int, float, int, int, hipStream_t);
void launch_branch_rmsnorm_add(const float*, float*, const void*, int64_t, int,
                               const void*, int64_t, float, float, const void*,
                               float, void*, int, int, int, hipStream_t);
void launch_clamped_glu(void*, const void*, int64_t, int, int, float, float,
                        int, hipStream_t);
void launch_mingru_scan(void*, const void*, int64_t, const float*, const float*,
                        float*, const int64_t*, const int*, const int*, int,
                        int, int, hipStream_t);
void launch_mingru_chunked(void*, float*, float*, const void*, int64_t,
                           const float*, const float*, float*, const int64_t*,
                           const int*, const int*, int, int, int, int, int,
                           hipStream_t);
}

static hipStream_t cur_stream() {
  return at::hip::getCurrentHIPStream().stream();
}

static int kind_of(const torch::Tensor& t, const char* what) {
  TORCH_CHECK(t.is_cuda(), what, " must be on the GPU");
  if (t.scalar_type() == at::kBFloat16) return 0;
  if (t.scalar_type() == at::kFloat) return 1;
  TORCH_CHECK(false, what, " must be bfloat16 or float32");
  return -1;
}

#define CHECK_I32(x) \
  TORCH_CHECK(x.is_cuda() && x.scalar_type() == at::kInt && x.is_contiguous(), #x " must be int32, contiguous, on the GPU")
#define CHECK_I64(x) \
  TORCH_CHECK(x.is_cuda() && x.scalar_type() == at::kLong && x.is_contiguous(), #x " must be int64, contiguous, on the GPU")
#define CHECK_F32C(x) \
  TORCH_CHECK(x.is_cuda() && x.scalar_type() == at::kFloat && x.is_contiguous(), #x " must be float32, contiguous, on the GPU")

// resid [T, W] fp32 (updated in place when y is given); y [T, W] (row stride
// free) or empty; scale [W]; weight/bias [W] or empty (no norm); out [T, W].
void add_layernorm(torch::Tensor resid, torch::Tensor y, torch::Tensor scale,
                   double mult, torch::Tensor weight, torch::Tensor bias,
                   double eps, torch::Tensor out) {
  CHECK_F32C(resid);
  TORCH_CHECK(resid.dim() == 2);
  const int rows = resid.size(0), W = resid.size(1);
  const bool has_y = y.numel() > 0, has_w = weight.numel() > 0;
  int y_kind = 1, p_kind = 1;
  int64_t y_stride = 0;
  if (has_y) {
    y_kind = kind_of(y, "y");
    TORCH_CHECK(y.dim() == 2 && y.size(0) == rows && y.size(1) == W &&
                y.stride(1) == 1);
    y_stride = y.stride(0);
    p_kind = kind_of(scale, "scale");
    TORCH_CHECK(scale.numel() == W && scale.is_contiguous());
  }
  if (has_w) {
    const int wk = kind_of(weight, "weight");
    TORCH_CHECK(!has_y || wk == p_kind, "scale and weight types differ");
    p_kind = wk;
    TORCH_CHECK(weight.numel() == W && bias.numel() == W &&
                weight.is_contiguous() && bias.is_contiguous() &&
                bias.scalar_type() == weight.scalar_type());
    TORCH_CHECK(out.is_cuda() && out.scalar_type() == weight.scalar_type() &&
                out.is_contiguous() && out.dim() == 2 && out.size(0) == rows &&
                out.size(1) == W);
  }
  launch_add_layernorm(resid.data_ptr<float>(),
                       has_y ? y.data_ptr() : nullptr, y_stride, y_kind,
                       has_y ? scale.data_ptr() : nullptr, (float)mult,
                       has_w ? weight.data_ptr() : nullptr,
                       has_w ? bias.data_ptr() : nullptr, (float)eps,
                       has_w ? out.data_ptr() : nullptr, p_kind, rows, W,
                       cur_stream());
}

// dkv [T, rank + rot_w]; cache [blocks, block, rank + rot_w]; freq [rot_dims/2]
void latent_kv_store(torch::Tensor dkv, torch::Tensor norm_w, double eps,
                     torch::Tensor freq, double mult, int64_t rot_dims,
                     torch::Tensor positions, torch::Tensor slots,
                     torch::Tensor cache, int64_t rank) {
  const int kind = kind_of(dkv, "dkv");
  TORCH_CHECK(dkv.dim() == 2 && dkv.stride(1) == 1);
  const int T = dkv.size(0);
  const int rot_w = dkv.size(1) - rank;
  TORCH_CHECK(rank > 0 && rot_w >= 0 && rot_dims % 2 == 0 && rot_dims <= rot_w);
  TORCH_CHECK(cache.is_cuda() && cache.scalar_type() == dkv.scalar_type() &&
              cache.is_contiguous() && cache.dim() == 3 &&
              cache.size(2) == rank + rot_w);
  TORCH_CHECK(norm_w.scalar_type() == dkv.scalar_type() &&
              norm_w.numel() == rank && norm_w.is_contiguous());
  CHECK_F32C(freq);
  TORCH_CHECK(freq.numel() == rot_dims / 2);
  CHECK_I32(positions);
  CHECK_I64(slots);
  TORCH_CHECK(positions.numel() == T && slots.numel() == T);
  launch_latent_kv_store(dkv.data_ptr(), dkv.stride(0), norm_w.data_ptr(),
                         (float)eps, freq.data_ptr<float>(), (float)mult,
                         (int)rot_dims, positions.data_ptr<int>(),
                         slots.data_ptr<int64_t>(), cache.data_ptr(), (int)rank,
                         rot_w, T, kind, cur_stream());
}

// q [T, H, D] (strided view); rotates columns [col0, col0 + rot_w) of every
// head into out [T, H, rot_w] fp32
void rope_rows(torch::Tensor out, torch::Tensor q, int64_t col0,
               torch::Tensor freq, double mult, int64_t rot_dims,
               torch::Tensor positions) {
  const int kind = kind_of(q, "q");
  CHECK_F32C(out);
  TORCH_CHECK(q.dim() == 3 && out.dim() == 3 && q.stride(2) == 1);
  const int T = q.size(0), H = q.size(1), rot_w = out.size(2);
  TORCH_CHECK(out.size(0) == T && out.size(1) == H);
  TORCH_CHECK(col0 >= 0 && col0 + rot_w <= q.size(2));
  TORCH_CHECK(rot_dims % 2 == 0 && rot_dims <= rot_w);
  CHECK_F32C(freq);
  TORCH_CHECK(freq.numel() == rot_dims / 2);
  CHECK_I32(positions);
  TORCH_CHECK(positions.numel() == T);
  launch_rope_rows(out.data_ptr<float>(), q.data_ptr(), q.stride(0),
                   q.stride(1), (int)col0, freq.data_ptr<float>(), (float)mult,
                   (int)rot_dims, positions.data_ptr<int>(), H, rot_w, T, kind,
                   cur_stream());
}

// out/q_lat [T, H, rank] fp32, q_rot [T, H, rot_w] fp32, cache [blocks, block,
// rank + rot_w], block_tables [B, max_blocks] int32, token_seq [T] int32 or
// empty (token i belongs to sequence i), positions [T] int32
void latent_window_attention(torch::Tensor out, torch::Tensor q_lat,
                             torch::Tensor q_rot, torch::Tensor cache,
                             torch::Tensor block_tables, torch::Tensor token_seq,
                             torch::Tensor positions, int64_t window,
                             double scale, int64_t max_keys) {
  const int kind = kind_of(cache, "cache");
  CHECK_F32C(out);
  CHECK_F32C(q_lat);
  CHECK_F32C(q_rot);
  TORCH_CHECK(q_lat.dim() == 3 && q_rot.dim() == 3 && cache.dim() == 3 &&
              cache.is_contiguous());
  const int T = q_lat.size(0), H = q_lat.size(1), rank = q_lat.size(2);
  const int rot_w = q_rot.size(2);
  TORCH_CHECK(q_rot.size(0) == T && q_rot.size(1) == H);
  TORCH_CHECK(out.sizes() == q_lat.sizes());
  TORCH_CHECK(cache.size(2) == rank + rot_w, "cache row width");
  TORCH_CHECK(rank <= 1024, "latent rank above 1024 is not supported");
  TORCH_CHECK(window >= 1);
  CHECK_I32(block_tables);
  CHECK_I32(positions);
  TORCH_CHECK(block_tables.dim() == 2 && positions.numel() == T);
  const bool has_seq = token_seq.numel() > 0;
  if (has_seq) {
    CHECK_I32(token_seq);
    TORCH_CHECK(token_seq.numel() == T);
  } else {
    TORCH_CHECK(block_tables.size(0) >= T);
  }
  // shares of the window per token: enough workgroups to fill the chip when
  // there are few tokens (decode). Only host-known sizes enter, so a captured
  // graph keeps its grid: max_keys is the longest context this launch can see.
  const int64_t keys = std::max<int64_t>(1, std::min<int64_t>(window, max_keys));
  const int64_t tiles_per_wg = 4;  // 64-key tiles, one per wave and round
  const int hb = rank <= 512 ? 8 : 4;
  const int64_t wgs = (int64_t)T * ((H + hb - 1) / hb);
  int splits = 1;
  if (wgs < 512) {
    const int64_t by_keys = (keys + 64 * tiles_per_wg - 1) / (64 * tiles_per_wg);
    const int64_t by_fill = (512 + wgs - 1) / wgs;
    splits = (int)std::max<int64_t>(1, std::min<int64_t>({by_keys, by_fill, 32}));
  }
  torch::Tensor part;
  if (splits > 1)
    part = torch::empty({(int64_t)T, H, splits, rank + 2}, q_lat.options());
  launch_latent_window_attention(
      out.data_ptr<float>(), splits > 1 ? part.data_ptr<float>() : nullptr,
      q_lat.data_ptr<float>(), q_rot.data_ptr<float>(), cache.data_ptr(),
      block_tables.data_ptr<int>(), (int)block_tables.stride(0),
      has_seq ? token_seq.data_ptr<int>() : nullptr, positions.data_ptr<int>(),
      T, H, rank, rot_w, (int)cache.size(1), (int)window, (float)scale, splits,
      kind, cur_stream());
}

// q, k, z [T, H*dk] and v [T, H*dv] (row strides free), z_bias [H*dk],
// state [slots, H, dk, dv] fp32, slots [B] int64, cu [B+1] int32 or empty (one
// token per sequence), positions [T] int32, o [T, H, dv] fp32
void gla_recurrence(torch::Tensor o, torch::Tensor q, torch::Tensor k,
                    torch::Tensor v, torch::Tensor z, torch::Tensor z_bias,
                    torch::Tensor state, torch::Tensor slots, torch::Tensor cu,
                    torch::Tensor positions, double inv_tau, double q_scale) {
  const int kind = kind_of(q, "q");
  CHECK_F32C(o);
  CHECK_F32C(state);
  TORCH_CHECK(state.dim() == 4 && o.dim() == 3);
  const int H = state.size(1), dk = state.size(2), dv = state.size(3);
  const int T = o.size(0);
  TORCH_CHECK(o.size(1) == H && o.size(2) == dv);
  TORCH_CHECK(dk <= 1024, "gla key dim above 1024 is not supported");
  for (const torch::Tensor* t : {&q, &k, &z}) {
    TORCH_CHECK(t->is_cuda() && t->scalar_type() == q.scalar_type() &&
                t->dim() == 2 && t->size(0) == T && t->size(1) == H * dk &&
                t->stride(1) == 1);
  }
  TORCH_CHECK(v.is_cuda() && v.scalar_type() == q.scalar_type() &&
              v.dim() == 2 && v.size(0) == T && v.size(1) == H * dv &&
              v.stride(1) == 1);
  TORCH_CHECK(z_bias.is_cuda() && z_bias.scalar_type() == q.scalar_type() &&
              z_bias.numel() == H * dk && z_bias.is_contiguous());
  CHECK_I64(slots);
  CHECK_I32(positions);
  TORCH_CHECK(positions.numel() == T);
  const int B = slots.numel();
  const bool has_cu = cu.numel() > 0;
  if (has_cu) {
    CHECK_I32(cu);
    TORCH_CHECK(cu.numel() == B + 1);
  } else {
    TORCH_CHECK(B == T, "without cu every sequence brings one token");
  }
  launch_gla_recurrence(
      o.data_ptr<float>(), q.data_ptr(), k.data_ptr(), v.data_ptr(),
      z.data_ptr(), q.stride(0), k.stride(0), v.stride(0), z.stride(0),
      z_bias.data_ptr(), state.data_ptr<float>(), slots.data_ptr<int64_t>(),
      has_cu ? cu.data_ptr<int>() : nullptr, positions.data_ptr<int>(), B, H,
      dk, dv, (float)inv_tau, (float)q_scale, kind, cur_stream());
}

// o [T, H, dv] fp32, gate [T, H*dv], weight [dv] -> out [T, H*dv]
void gated_rmsnorm(torch::Tensor out, torch::Tensor o, torch::Tensor gate,
                   torch::Tensor weight, double eps) {
  const int kind = kind_of(gate, "gate");
  CHECK_F32C(o);
  TORCH_CHECK(o.dim() == 3);
  const int T = o.size(0), H = o.size(1), dv = o.size(2);
  TORCH_CHECK(gate.dim() == 2 && gate.size(0) == T && gate.size(1) == H * dv &&
              gate.stride(1) == 1);
  TORCH_CHECK(out.is_cuda() && out.scalar_type() == gate.scalar_type() &&
              out.is_contiguous() && out.numel() == (int64_t)T * H * dv);
  TORCH_CHECK(weight.is_cuda() && weight.scalar_type() == gate.scalar_type() &&
              weight.numel() == dv && weight.is_contiguous());
  launch_gated_rmsnorm(out.data_ptr(), o.data_ptr<float>(), gate.data_ptr(),
                       gate.stride(0), weight.data_ptr(), (float)eps, T * H, H,
                       dv, kind, cur_stream());
}

// x [T, W] fp32 (in place); y [T, W] (row stride free) + w_branch [W] or
// empty; hist [n_max, T, W] fp32 or empty; dwa [n_hist] fp32 or empty; w_next
// [W] + out [T, W] or empty; add_table [N, W] + add_index [T] int32 or empty
void sandwich_rmsnorm(torch::Tensor x, torch::Tensor y, torch::Tensor w_branch,
                      torch::Tensor hist, int64_t n_hist, torch::Tensor dwa,
                      torch::Tensor w_next, double eps, double offset,
                      torch::Tensor out, torch::Tensor add_table,
                      torch::Tensor add_index) {
  CHECK_F32C(x);
  TORCH_CHECK(x.dim() == 2);
  const int rows = x.size(0), W = x.size(1);
  const bool has_y = y.numel() > 0, has_n = w_next.numel() > 0;
  const bool has_h = hist.numel() > 0, has_d = dwa.numel() > 0;
  const bool has_t = add_table.numel() > 0;
  int y_kind = 1, p_kind = -1;
  int64_t y_stride = 0;
  auto param = [&](const torch::Tensor& t, const char* what) {
    const int k = kind_of(t, what);
    TORCH_CHECK(p_kind < 0 || k == p_kind, "parameter types differ");
    p_kind = k;
  };
  if (has_y) {
    y_kind = kind_of(y, "y");
    TORCH_CHECK(y.dim() == 2 && y.size(0) == rows && y.size(1) == W &&
                y.stride(1) == 1);
    y_stride = y.stride(0);
    param(w_branch, "w_branch");
    TORCH_CHECK(w_branch.numel() == W && w_branch.is_contiguous());
  }
  if (has_n) {
    param(w_next, "w_next");
    TORCH_CHECK(w_next.numel() == W && w_next.is_contiguous());
    TORCH_CHECK(out.is_cuda() && out.scalar_type() == w_next.scalar_type() &&
                out.is_contiguous() && out.dim() == 2 && out.size(0) == rows &&
                out.size(1) == W);
  }
  if (has_t) {
    param(add_table, "add_table");
    TORCH_CHECK(add_table.dim() == 2 && add_table.size(1) == W &&
                add_table.is_contiguous());
    CHECK_I32(add_index);
    TORCH_CHECK(add_index.numel() == rows);
  }
  if (has_h) {
    CHECK_F32C(hist);
    TORCH_CHECK(hist.dim() == 3 && hist.size(1) == rows && hist.size(2) == W);
    TORCH_CHECK(n_hist >= 1 && n_hist <= hist.size(0));
  }
  if (has_d) {
    CHECK_F32C(dwa);
    TORCH_CHECK(has_h && dwa.numel() == n_hist);
  }
  if (p_kind < 0) p_kind = 1;
  launch_sandwich_rmsnorm(
      x.data_ptr<float>(), has_y ? y.data_ptr() : nullptr, y_stride, y_kind,
      has_y ? w_branch.data_ptr() : nullptr,
      has_h ? hist.data_ptr<float>() : nullptr, (int64_t)rows * W, (int)n_hist,
      has_d ? dwa.data_ptr<float>() : nullptr,
      has_n ? w_next.data_ptr() : nullptr, (float)eps, (float)offset,
      has_n ? out.data_ptr() : nullptr, has_t ? add_table.data_ptr() : nullptr,
      has_t ? add_index.data_ptr<int>() : nullptr, p_kind, rows, W,
      cur_stream());
}

void xielu(torch::Tensor out, torch::Tensor x, double a_pos, double a_neg) {
  const int kind = kind_of(x, "x");
  TORCH_CHECK(x.is_contiguous() && out.is_cuda() && out.is_contiguous() &&
              out.scalar_type() == x.scalar_type() && out.numel() == x.numel());
  launch_xielu(out.data_ptr(), x.data_ptr(), x.numel(), (float)a_pos,
               (float)a_neg, kind, cur_stream());
}

// q [T, wq], k [T, wk] or empty, v [T, wv] or empty (values = k) — row strides
// free; q_out [T, wq] fp32; cache [blocks, block, wk + wv]
void qkv_store(torch::Tensor q_out, torch::Tensor q, torch::Tensor k,
               torch::Tensor v, torch::Tensor positions, torch::Tensor slots,
               torch::Tensor cache, int64_t seg, double eps, double temp_coef,
               int64_t temp_every, torch::Tensor q_weight,
               torch::Tensor k_weight, torch::Tensor rot_freq, double rot_mult,
               int64_t rot_dims, bool norm_whole, bool rot_interleaved,
               torch::Tensor v_rot_freq, int64_t v_seg, torch::Tensor v_cs_out) {
  const int kind = kind_of(q, "q");
  const bool has_qw = q_weight.numel() > 0, has_kw = k_weight.numel() > 0;
  const bool has_rot = rot_freq.numel() > 0 && rot_dims > 0;
  const bool has_vrot = v_rot_freq.numel() > 0;
  if (has_qw || has_kw || has_rot)
    TORCH_CHECK(seg > 0 && q.size(1) % seg == 0, "query width / segment");
  // norm_whole: the RMS runs over the whole row and so do the weights
  if (has_qw) {
    CHECK_F32C(q_weight);
    TORCH_CHECK(q_weight.numel() == (norm_whole ? q.size(1) : seg),
                "query norm weight width");
  }
  if (has_kw) {
    CHECK_F32C(k_weight);
    TORCH_CHECK(k.dim() == 2 &&
                k_weight.numel() == (norm_whole ? k.size(1) : seg),
                "key norm weight width");
  }
  // v_cs_out [T, v_seg] fp32: the tokens' (cos, sin) pairs of that rotation
  const bool has_vcs = has_vrot && v_cs_out.numel() > 0;
  if (has_vrot) {
    CHECK_F32C(v_rot_freq);
    TORCH_CHECK(v_seg > 0 && v_seg % 2 == 0 && v_rot_freq.numel() == v_seg / 2 &&
                (v.dim() != 2 || v.size(1) % v_seg == 0),
                "rotated value segments");
  }
  if (has_vcs) {
    CHECK_F32C(v_cs_out);
    TORCH_CHECK(v_cs_out.numel() == q.size(0) * v_seg, "cos/sin table size");
  }
  if (has_rot) {
    CHECK_F32C(rot_freq);
    TORCH_CHECK(rot_dims % 2 == 0 && rot_dims <= seg &&
                rot_freq.numel() == rot_dims / 2, "rotated dimensions");
  }
  CHECK_F32C(q_out);
  TORCH_CHECK(q.dim() == 2 && q.stride(1) == 1 && q_out.dim() == 2);
  const int T = q.size(0), wq = q.size(1);
  TORCH_CHECK(q_out.size(0) == T && q_out.size(1) == wq);
  CHECK_I32(positions);
  TORCH_CHECK(positions.numel() == T);
  const bool has_k = k.dim() == 2;
  const bool has_v = v.numel() > 0;
  int wk = 0, wv = 0;
  if (eps >= 0) TORCH_CHECK(seg > 0 && wq % seg == 0, "query width / segment");
  if (has_k) {
    TORCH_CHECK(k.is_cuda() && k.scalar_type() == q.scalar_type() &&
                k.dim() == 2 && k.size(0) == T && k.stride(1) == 1);
    wk = k.size(1);
    if (eps >= 0 || has_kw || has_rot)
      TORCH_CHECK(wk % seg == 0, "key width / segment");
    if (has_v) {
      TORCH_CHECK(v.is_cuda() && v.scalar_type() == q.scalar_type() &&
                  v.dim() == 2 && v.size(0) == T && v.stride(1) == 1);
      wv = v.size(1);
    } else {
      wv = wk;
    }
    TORCH_CHECK(cache.is_cuda() && cache.scalar_type() == q.scalar_type() &&
                cache.is_contiguous() && cache.dim() == 3 &&
                cache.size(2) == wk + wv, "cache row width");
    CHECK_I64(slots);
    TORCH_CHECK(slots.numel() == T);
  }
  launch_qkv_store(q_out.data_ptr<float>(), q.data_ptr(), q.stride(0),
                   has_k ? k.data_ptr() : nullptr, has_k ? k.stride(0) : 0,
                   has_v ? v.data_ptr() : nullptr, has_v ? v.stride(0) : 0,
                   positions.data_ptr<int>(),
                   has_k ? slots.data_ptr<int64_t>() : nullptr,
                   has_k ? cache.data_ptr() : nullptr, wq, wk, wv, (int)seg,
                   (float)eps, (float)temp_coef, (int)temp_every,
                   has_qw ? q_weight.data_ptr<float>() : nullptr,
                   has_kw ? k_weight.data_ptr<float>() : nullptr,
                   has_rot ? rot_freq.data_ptr<float>() : nullptr,
                   (float)rot_mult, has_rot ? (int)rot_dims : 0,
                   norm_whole ? 1 : 0, rot_interleaved ? 1 : 0,
                   has_vrot ? v_rot_freq.data_ptr<float>() : nullptr,
                   has_vrot ? (int)v_seg : 0,
                   has_vcs ? v_cs_out.data_ptr<float>() : nullptr, T, kind,
                   cur_stream());
}

// cache [blocks, block, E]; pool [blocks, per_page, E] fp32
void pool_cache_update(torch::Tensor cache, torch::Tensor pool,
                       torch::Tensor block_tables, torch::Tensor token_seq,
                       torch::Tensor positions, torch::Tensor slots, int64_t P) {
  const int kind = kind_of(cache, "cache");
  CHECK_F32C(pool);
  TORCH_CHECK(cache.dim() == 3 && cache.is_contiguous() && pool.dim() == 3);
  const int E = cache.size(2), bs = cache.size(1), per_page = pool.size(1);
  TORCH_CHECK(P >= 1 && pool.size(2) == E && pool.size(0) == cache.size(0));
  TORCH_CHECK((int64_t)per_page * P >= bs, "pooled rows per page");
  CHECK_I32(block_tables);
  CHECK_I32(positions);
  CHECK_I64(slots);
  const int T = positions.numel();
  TORCH_CHECK(block_tables.dim() == 2 && slots.numel() == T);
  const bool has_seq = token_seq.numel() > 0;
  if (has_seq) {
    CHECK_I32(token_seq);
    TORCH_CHECK(token_seq.numel() == T);
  } else {
    TORCH_CHECK(block_tables.size(0) >= T);
  }
  launch_pool_cache_update(cache.data_ptr(), pool.data_ptr<float>(),
                           block_tables.data_ptr<int>(),
                           (int)block_tables.stride(0),
                           has_seq ? token_seq.data_ptr<int>() : nullptr,
                           positions.data_ptr<int>(), slots.data_ptr<int64_t>(),
                           E, bs, per_page, (int)P, T, kind, cur_stream());
}

// out [T, H * dv] (cache type), q [T, H * M * d] fp32, cache [blocks, block,
// G * M * d + G * dv], pool [blocks, per_page, same width] fp32 or empty
void row_attention(torch::Tensor out, torch::Tensor q, torch::Tensor cache,
                   torch::Tensor pool, torch::Tensor block_tables,
                   torch::Tensor token_seq, torch::Tensor positions, int64_t H,
                   int64_t G, int64_t M, int64_t d, int64_t dv, int64_t window,
                   int64_t P, double scale, double softcap, double lam,
                   double norm_eps, double out_mult, int64_t max_keys,
                   torch::Tensor query_bounds, torch::Tensor head_bias,
                   torch::Tensor gate, int64_t value_col, torch::Tensor rot_cs,
                   bool rot_interleaved) {
  const int kind = kind_of(cache, "cache");
  CHECK_F32C(q);
  // head_bias [H] fp32: sigmoid(score + head_bias[h]) weights, not normalised;
  // gate [T, H] (cache type, row stride free): result times sigmoid(gate)
  const bool has_bias = head_bias.numel() > 0, has_gate = gate.numel() > 0;
  if (has_bias) {
    CHECK_F32C(head_bias);
    TORCH_CHECK(head_bias.numel() == H && M == 1, "head bias");
  }
  if (has_gate)
    TORCH_CHECK(gate.is_cuda() && gate.scalar_type() == cache.scalar_type() &&
                gate.dim() == 2 && gate.size(0) == q.size(0) &&
                gate.size(1) == H && gate.stride(1) == 1, "gate");
  const float* bias_p = has_bias ? head_bias.data_ptr<float>() : nullptr;
  const void* gate_p = has_gate ? gate.data_ptr() : nullptr;
  const int64_t gate_stride = has_gate ? gate.stride(0) : 0;
  TORCH_CHECK(q.dim() == 2 && cache.dim() == 3 && cache.is_contiguous());
  const int T = q.size(0);
  TORCH_CHECK(H >= 1 && G >= 1 && H % G == 0 && (M == 1 || M == 2) && d >= 1 &&
              dv >= 1);
  TORCH_CHECK(dv <= 256, "value width above 256 is not supported");
  TORCH_CHECK(d <= 1024, "key width above 1024 is not supported");
  TORCH_CHECK(q.size(1) == H * M * d, "query width");
  // value_col < 0: a row is [keys | values]. value_col >= 0: a row holds the
  // keys only and the values are its columns from value_col on (0 with dv ==
  // d: the values ARE the keys; other columns: a share of a wide latent row)
  if (value_col >= 0)
    TORCH_CHECK(M == 1 && G == 1 && value_col + dv <= d, "shared keys and values");
  const int vbase = value_col >= 0 ? (int)value_col : (int)(G * M * d);
  const int E = std::max<int>((int)(G * M * d), vbase + (int)(G * dv));
  TORCH_CHECK(cache.size(2) == E, "cache row width");
  // the result has the cache's type, or fp32
  TORCH_CHECK(out.is_cuda() && (out.scalar_type() == cache.scalar_type() ||
                                out.scalar_type() == torch::kFloat32) &&
              out.is_contiguous() && out.dim() == 2 && out.size(0) == T &&
              out.size(1) == H * dv);
  float* out32 = (kind == 0 && out.scalar_type() == torch::kFloat32)
                     ? out.data_ptr<float>() : nullptr;
  // rot_cs [T, dv / 2][2] fp32 (cos, sin per token and pair): every head's
  // result is turned back by its token's angles
  const bool has_rot = rot_cs.numel() > 0;
  if (has_rot) {
    CHECK_F32C(rot_cs);
    TORCH_CHECK(dv % 2 == 0 && rot_cs.numel() == (int64_t)T * dv,
                "cos/sin table size");
  }
  const float* rot_p = has_rot ? rot_cs.data_ptr<float>() : nullptr;
  const int rot_inter = rot_interleaved ? 1 : 0;
  TORCH_CHECK(window >= 0 && P >= 0);
  int per_page = 1;
  const bool has_pool = window > 0 && P > 0;
  if (has_pool) {
    CHECK_F32C(pool);
    TORCH_CHECK(pool.dim() == 3 && pool.size(2) == E &&
                pool.size(0) == cache.size(0));
    per_page = pool.size(1);
    TORCH_CHECK((int64_t)per_page * P >= cache.size(1), "pooled rows per page");
  }
  CHECK_I32(block_tables);
  CHECK_I32(positions);
  TORCH_CHECK(block_tables.dim() == 2 && positions.numel() == T);
  const bool has_seq = token_seq.numel() > 0;
  if (has_seq) {
    CHECK_I32(token_seq);
    TORCH_CHECK(token_seq.numel() == T);
  } else {
    TORCH_CHECK(block_tables.size(0) >= T);
  }
  // prompt portions (token bounds per sequence given, tokens of a sequence
  // consecutive): the matrix-core kernel, 32 tokens per workgroup
  if (query_bounds.numel() > 0 && has_seq &&
      row_attention_prefill_supported((int)d, (int)dv)) {
    CHECK_I32(query_bounds);
    const int B = query_bounds.numel() - 1;
    TORCH_CHECK(B >= 1 && block_tables.size(0) >= B);
    // a value width that does not fill its tile cannot pair halves in
    // registers: fp32 results, then a pass of its own turns them
    const bool turn_after =
        has_rot && !row_attention_prefill_rotates((int)dv, rot_inter);
    torch::Tensor tmp;
    void* out_p = out.data_ptr();
    float* out32_p = out32;
    if (turn_after) {
      tmp = torch::empty({(int64_t)T, H * dv}, q.options());
      out_p = tmp.data_ptr();
      out32_p = kind == 0 ? tmp.data_ptr<float>() : nullptr;
    }
    launch_row_attention_prefill(
        out_p, out32_p, q.data_ptr<float>(), cache.data_ptr(),
        has_pool ? pool.data_ptr<float>() : nullptr,
        block_tables.data_ptr<int>(), (int)block_tables.stride(0),
        query_bounds.data_ptr<int>(), B, positions.data_ptr<int>(),
        (T + 31) / 32 + B, (int)H, (int)G, (int)M, (int)d, (int)dv,
        (int)cache.size(1), per_page, (int)window, has_pool ? (int)P : 0,
        (float)scale, (float)softcap, (float)lam, (float)norm_eps,
        (float)out_mult, bias_p, gate_p, gate_stride, vbase,
        turn_after ? nullptr : rot_p, rot_inter, kind, cur_stream());
    if (turn_after)
      launch_rotate_heads_table(out.data_ptr(), tmp.data_ptr<float>(), rot_p,
                                (int)H, (int)dv, rot_inter, -1.0f, T,
                                kind_of(out, "out"), cur_stream());
    return;
  }
  // shares of the key list per token: enough workgroups to fill the chip
  // when there are few tokens (decode). Only host-known sizes enter, so a
  // captured graph keeps its grid.
  int64_t keys = std::max<int64_t>(1, max_keys);
  if (window > 0) {
    const int64_t beyond = std::max<int64_t>(0, keys - window);
    keys = std::min<int64_t>(keys, window) + (has_pool ? beyond / P : 0);
  }
  const int rep = H / G;
  const int hb = row_attention_heads_per_group(rep);
  const int64_t wgs = (int64_t)T * G * ((rep + hb - 1) / hb);
  int splits = 1;
  if (wgs < 512) {
    const int64_t by_keys = (keys + 255) / 256;  // 4 waves x 64 keys per pass
    const int64_t by_fill = (512 + wgs - 1) / std::max<int64_t>(1, wgs);
    splits = (int)std::max<int64_t>(1, std::min<int64_t>({by_keys, by_fill, 32}));
  }
  torch::Tensor part;
  if (splits > 1)
    part = torch::empty({(int64_t)T, H, splits, M, dv + 2}, q.options());
  launch_row_attention(
      out.data_ptr(), out32, splits > 1 ? part.data_ptr<float>() : nullptr,
      q.data_ptr<float>(), cache.data_ptr(),
      has_pool ? pool.data_ptr<float>() : nullptr, block_tables.data_ptr<int>(),
      (int)block_tables.stride(0), has_seq ? token_seq.data_ptr<int>() : nullptr,
      positions.data_ptr<int>(), T, (int)H, (int)G, (int)M, (int)d, (int)dv,
      (int)cache.size(1), per_page, (int)window, has_pool ? (int)P : 0,
      (float)scale, (float)softcap, (float)lam, (float)norm_eps,
      (float)out_mult, splits, bias_p, gate_p, gate_stride, vbase, rot_p,
      rot_inter, kind, cur_stream());
}

// x [T, W] fp32 (updated in place when y1 is given); y1, y2 [T, W] of the
// activation type or empty (row strides free); weight [W] and out [T, W] of
// the activation type, or both empty (no norm)
void group_rmsnorm_add(torch::Tensor x, torch::Tensor y1, torch::Tensor y2,
                       torch::Tensor weight, int64_t groups, double eps,
                       torch::Tensor out) {
  CHECK_F32C(x);
  TORCH_CHECK(x.dim() == 2);
  const int T = x.size(0), W = x.size(1);
  const bool has_y1 = y1.numel() > 0, has_y2 = y2.numel() > 0;
  const bool has_w = weight.numel() > 0;
  TORCH_CHECK(has_y1 || has_w, "nothing to do");
  TORCH_CHECK(has_y1 || !has_y2, "y2 without y1");
  const int kind = kind_of(has_w ? weight : y1, "activation");
  auto check_y = [&](const torch::Tensor& y) {
    TORCH_CHECK(y.is_cuda() && kind_of(y, "y") == kind && y.dim() == 2 &&
                y.size(0) == T && y.size(1) == W && y.stride(1) == 1);
  };
  if (has_y1) check_y(y1);
  if (has_y2) check_y(y2);
  TORCH_CHECK(groups >= 1 && groups <= 1024 && W % groups == 0,
              "the width does not split into the norm's groups");
  if (has_w)
    TORCH_CHECK(weight.is_cuda() && weight.is_contiguous() &&
                weight.numel() == W && out.is_cuda() && out.is_contiguous() &&
                kind_of(out, "out") == kind && out.dim() == 2 &&
                out.size(0) == T && out.size(1) == W);
  launch_group_rmsnorm_add(x.data_ptr<float>(),
                           has_y1 ? y1.data_ptr() : nullptr,
                           has_y1 ? y1.stride(0) : 0,
                           has_y2 ? y2.data_ptr() : nullptr,
                           has_y2 ? y2.stride(0) : 0,
                           has_w ? weight.data_ptr() : nullptr, (float)eps,
                           has_w ? out.data_ptr() : nullptr, T, W, (int)groups,
                           kind, cur_stream());
}

// out [T, W] fp32; ids, prev [T] int64; table [vocab, W], pair [buckets + 1, W]
void pair_hash_embedding(torch::Tensor out, torch::Tensor ids,
                         torch::Tensor prev, torch::Tensor table,
                         torch::Tensor pair, double scale, int64_t buckets,
                         int64_t mul_prev, int64_t mul_cur) {
  const int kind = kind_of(table, "table");
  CHECK_F32C(out);
  CHECK_I64(ids);
  CHECK_I64(prev);
  const int T = ids.numel(), W = table.size(1);
  TORCH_CHECK(prev.numel() == T && out.dim() == 2 && out.size(0) == T &&
              out.size(1) == W);
  TORCH_CHECK(table.dim() == 2 && table.is_contiguous() && pair.is_cuda() &&
              pair.scalar_type() == table.scalar_type() && pair.dim() == 2 &&
              pair.is_contiguous() && pair.size(1) == W &&
              pair.size(0) == buckets + 1 && buckets >= 1, "pair table");
  launch_pair_hash_embedding(out.data_ptr<float>(), ids.data_ptr<int64_t>(),
                             prev.data_ptr<int64_t>(), table.data_ptr(),
                             pair.data_ptr(), (float)scale, buckets, mul_prev,
                             mul_cur, table.size(0), W, T, kind, cur_stream());
}

// x [rows, I] (row stride free) -> out [rows, I]
void relu_squared(torch::Tensor out, torch::Tensor x) {
  const int kind = kind_of(x, "x");
  TORCH_CHECK(x.dim() == 2 && x.stride(1) == 1 && out.is_cuda() &&
              out.scalar_type() == x.scalar_type() && out.is_contiguous() &&
              out.dim() == 2 && out.size(0) == x.size(0) &&
              out.size(1) == x.size(1));
  launch_relu_squared(out.data_ptr(), x.data_ptr(), x.stride(0), (int)x.size(1),
                      (int)x.size(0), kind, cur_stream());
}

// x [T, H, D] fp32 -> out [T, H * D] (bf16 or fp32); freq [D / 2]
void rotate_heads(torch::Tensor out, torch::Tensor x, torch::Tensor freq,
                  torch::Tensor positions, bool interleaved, double sign) {
  const int kind = kind_of(out, "out");
  CHECK_F32C(x);
  CHECK_F32C(freq);
  CHECK_I32(positions);
  TORCH_CHECK(x.dim() == 3);
  const int T = x.size(0), H = x.size(1), D = x.size(2);
  TORCH_CHECK(D % 2 == 0 && freq.numel() == D / 2 && positions.numel() == T);
  TORCH_CHECK(out.is_contiguous() && out.dim() == 2 && out.size(0) == T &&
              out.size(1) == (int64_t)H * D);
  launch_rotate_heads(out.data_ptr(), x.data_ptr<float>(),
                      freq.data_ptr<float>(), positions.data_ptr<int>(), H, D,
                      interleaved ? 1 : 0, (float)sign, T, kind, cur_stream());
}

// x_in [T, W] fp32 or empty; x_out [T, W] fp32 or empty (may be x_in); y1
// [T, W] activation type or fp32, y2 [T, W] activation type or empty (row
// strides free); weight [W] and out [T, W] of the activation type
void branch_rmsnorm_add(torch::Tensor x_in, torch::Tensor x_out,
                        torch::Tensor y1, torch::Tensor y2, double a, double b,
                        torch::Tensor weight, double eps, torch::Tensor out) {
  const int kind = kind_of(out, "out");
  const int y1_kind = kind_of(y1, "y1");
  TORCH_CHECK(y1.dim() == 2 && y1.stride(1) == 1 && out.dim() == 2 &&
              out.is_contiguous());
  const int T = y1.size(0), W = y1.size(1);
  TORCH_CHECK(out.size(0) == T && out.size(1) == W);
  TORCH_CHECK(kind == 0 || y1_kind == 1, "fp32 stacks take fp32 branches");
  TORCH_CHECK(weight.is_cuda() && weight.scalar_type() == out.scalar_type() &&
              weight.is_contiguous() && weight.numel() == W, "norm weight");
  const bool has_x = x_in.numel() > 0, has_o = x_out.numel() > 0;
  if (has_x) {
    CHECK_F32C(x_in);
    TORCH_CHECK(x_in.dim() == 2 && x_in.size(0) == T && x_in.size(1) == W);
  }
  if (has_o) {
    CHECK_F32C(x_out);
    TORCH_CHECK(x_out.dim() == 2 && x_out.size(0) == T && x_out.size(1) == W);
  }
  const bool has_y2 = y2.numel() > 0;
  if (has_y2)
    TORCH_CHECK(y2.is_cuda() && y2.scalar_type() == out.scalar_type() &&
                y2.dim() == 2 && y2.size(0) == T && y2.size(1) == W &&
                y2.stride(1) == 1, "second branch");
  launch_branch_rmsnorm_add(
      has_x ? x_in.data_ptr<float>() : nullptr,
      has_o ? x_out.data_ptr<float>() : nullptr, y1.data_ptr(), y1.stride(0),
      y1_kind, has_y2 ? y2.data_ptr() : nullptr, has_y2 ? y2.stride(0) : 0,
      (float)a, (float)b, weight.data_ptr(), (float)eps, out.data_ptr(), T, W,
      kind, cur_stream());
}

// x [T, 2 I] (row stride free) -> out [T, I]
void clamped_glu(torch::Tensor out, torch::Tensor x, double limit, double alpha) {
  const int kind = kind_of(x, "x");
  TORCH_CHECK(x.dim() == 2 && x.stride(1) == 1 && x.size(1) % 2 == 0);
  const int T = x.size(0), I = x.size(1) / 2;
  TORCH_CHECK(out.is_cuda() && out.scalar_type() == x.scalar_type() &&
              out.is_contiguous() && out.dim() == 2 && out.size(0) == T &&
              out.size(1) == I);
  launch_clamped_glu(out.data_ptr(), x.data_ptr(), x.stride(0), T, I,
                     (float)limit, (float)alpha, kind, cur_stream());
}

// zug [T, 3 width] (row stride free); state [slots, width] fp32; slots [B]
// int64; cu [B + 1] int32 or empty (one token per sequence); out [T, width]
void mingru_scan(torch::Tensor out, torch::Tensor zug, torch::Tensor z_bias,
                 torch::Tensor u_bias, torch::Tensor state, torch::Tensor slots,
                 torch::Tensor cu, torch::Tensor positions) {
  const int kind = kind_of(zug, "zug");
  CHECK_F32C(z_bias);
  CHECK_F32C(u_bias);
  CHECK_F32C(state);
  CHECK_I64(slots);
  CHECK_I32(positions);
  TORCH_CHECK(state.dim() == 2 && zug.dim() == 2 && zug.stride(1) == 1);
  const int T = zug.size(0), width = state.size(1);
  TORCH_CHECK(zug.size(1) == 3 * width && z_bias.numel() == width &&
              u_bias.numel() == width, "minGRU widths");
  TORCH_CHECK(out.is_cuda() && out.scalar_type() == zug.scalar_type() &&
              out.is_contiguous() && out.dim() == 2 && out.size(0) == T &&
              out.size(1) == width);
  TORCH_CHECK(positions.numel() == T);
  const int B = slots.numel();
  const bool has_cu = cu.numel() > 0;
  if (has_cu) {
    CHECK_I32(cu);
    TORCH_CHECK(cu.numel() == B + 1);
  } else {
    TORCH_CHECK(B == T, "one token per sequence without token bounds");
  }
  // long prompt portions: chunks of L tokens side by side (about 64 chunks
  // for a sequence of average length at most, so that folding the earlier
  // chunks stays cheap)
  if (has_cu && T >= 256) {
    const int per_seq = (T + B - 1) / B;
    const int L = std::max(64, ((per_seq + 63) / 64 + 7) / 8 * 8);
    const int tiles = (T + L - 1) / L + B;
    torch::Tensor carry = torch::empty({(int64_t)tiles, 2, width}, state.options());
    torch::Tensor init = torch::empty({(int64_t)B, width}, state.options());
    launch_mingru_chunked(out.data_ptr(), carry.data_ptr<float>(),
                          init.data_ptr<float>(), zug.data_ptr(), zug.stride(0),
                          z_bias.data_ptr<float>(), u_bias.data_ptr<float>(),
                          state.data_ptr<float>(), slots.data_ptr<int64_t>(),
                          cu.data_ptr<int>(), positions.data_ptr<int>(), B, L,
                          tiles, width, kind, cur_stream());
    return;
  }
  launch_mingru_scan(out.data_ptr(), zug.data_ptr(), zug.stride(0),
                     z_bias.data_ptr<float>(), u_bias.data_ptr<float>(),
                     state.data_ptr<float>(), slots.data_ptr<int64_t>(),
                     has_cu ? cu.data_ptr<int>() : nullptr,
                     positions.data_ptr<int>(), B, width, kind, cur_stream());
}

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.def("add_layernorm", &add_layernorm);
  m.def("latent_kv_store", &latent_kv_store);
  m.def("rope_rows", &rope_rows);
  m.def("latent_window_attention", &latent_window_attention);
  m.def("gla_recurrence", &gla_recurrence);
  m.def("gated_rmsnorm", &gated_rmsnorm);
  m.def("sandwich_rmsnorm", &sandwich_rmsnorm);
  m.def("xielu", &xielu);
  m.def("qkv_store", &qkv_store);
  m.def("pool_cache_update", &pool_cache_update);
  m.def("row_attention", &row_attention);
  m.def("branch_rmsnorm_add", &branch_rmsnorm_add);
  m.def("clamped_glu", &clamped_glu);
  m.def("mingru_scan", &mingru_scan);
  m.def("group_rmsnorm_add", &group_rmsnorm_add);
  m.def("pair_hash_embedding", &pair_hash_embedding);
  m.def("relu_squared", &relu_squared);
  m.def("rotate_heads", &rotate_heads);
}
