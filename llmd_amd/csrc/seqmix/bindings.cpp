// Python bindings of the sequence-mixer op library (llmd_amd._C_seqmix). Host C++ only; the
// kernels live in the sm_*.hip units behind extern "C" launchers. Every binding checks device,
// dtype, contiguity and the shapes its kernel's grid assumes, so a bad call raises instead of
// faulting the GPU. Activations are bfloat16 or float32 (f32 flag), never mixed in one call.
#include <torch/extension.h>
#include <c10/hip/HIPGuard.h>
#include <c10/hip/HIPStream.h>
#include <hip/hip_runtime.h>

extern "C" {
void sm_embed_scale(const int64_t*, const void*, float, float*, float*, int, int, int64_t, int, hipStream_t);
void sm_zc_norm(const float*, const void*, float, void*, int, int, int, hipStream_t);
void sm_add_post_norm(const void*, int64_t, const void*, const void*, float*, float, const void*, void*, int, int, int,
                      hipStream_t);
void sm_depth_avg_norm(float*, int64_t, int, const float*, int, const void*, float, void*, int, int, int, hipStream_t);
void sm_xielu(const void*, float, float, void*, int64_t, int, hipStream_t);
void sm_softcap(float*, float, int64_t, hipStream_t);
void sm_latent_rope_cache(const void*, int64_t, const void*, int64_t, const void*, float, const int64_t*, const float*,
                          int, int, int, int, int, const int64_t*, void*, void*, int, int, int, hipStream_t);
int sm_latent_attention(const void*, const void*, const int*, int, int, const int*, const int*, float, int, int, int,
                        int, int, void*, int, const void*, int64_t, hipStream_t);
int sm_latent_attention_mfma(const void*, const void*, const int*, int, int, const int*, int, const int*, float, int,
                             int, int, void*, int, int, float*, float*, const void*, int64_t, hipStream_t);
void sm_embed_norm(const int64_t*, const void*, int64_t, const void*, float, float*, void*, int, int, int, hipStream_t);
void sm_rms_norm_rows(const void*, int64_t, const void*, float, void*, int, int, int, hipStream_t);
void sm_relu2(const void*, void*, int64_t, int, hipStream_t);
void sm_input_conv(const void*, int, const void*, int, void*, const int*, const int*, const int*, const int*, void*,
                   int, int, int, int, hipStream_t);
int sm_hgrn2_scan(const void*, int64_t, int, int, int, const float*, const float*, const void*, float, float*,
                  const int*, const int*, const int*, void*, float*, float*, float*, float*, int, int, int, int,
                  const int*, const int*, const int*, const int*, const int*, float*, float*, hipStream_t);
void sm_causal_conv_silu(const void*, int64_t, int, const void*, const void*, int, void*, const int*, const int*,
                         const int*, void*, int, int, int, hipStream_t);
int sm_selective_scan(const void*, const void*, const void*, const float*, const void*, int64_t, int, int, const void*,
                      const void*, int64_t, int, float*, const int*, const int*, const int*, void*, int, int,
                      hipStream_t);
int sm_gdelta_scan(const void*, int64_t, const void*, const void*, const void*, const void*, float, int, int, float*,
                   const int*, const int*, const int*, void*, int, int, hipStream_t);
void sm_hyper_embed(const int64_t*, const void*, int64_t, float*, int, int, int, int, hipStream_t);
void sm_hyper_norm(const float*, const float*, const void*, float, void*, int, int, int, int, hipStream_t);
void sm_hyper_update_norm(float*, const void*, int64_t, const float*, const float*, const float*, const void*, float,
                          void*, int, int, int, int, hipStream_t);
void sm_gated_act(const void*, int64_t, int, int, void*, int, int, hipStream_t);
void sm_qkv_rope_cache(const void*, int64_t, const float*, const int64_t*, const float*, int, int, int, int, int, int,
                       int, float, float*, int, float, const int64_t*, void*, int, void*, const float*, int, int, int,
                       int, hipStream_t);
int sm_grouped_attention(const void*, const void*, const int*, int, int, const int*, const int*, float, int, int, int,
                         int, int, int, const void*, int64_t, void*, int, const float*, int, const float*, int, int,
                         hipStream_t);
int sm_grouped_attention_mfma(const void*, const void*, const int*, int, int, const int*, int, const int*, float, int,
                              int, int, int, const void*, int64_t, void*, int, int, float*, float*, int, const float*,
                              int, const float*, int, int, hipStream_t);
void sm_moe_route_scores(const float*, const float*, int, int, int*, float*, int, hipStream_t);
void sm_moe_route(const float*, int, int, int*, float*, int, int, hipStream_t);
void sm_moe_group(const int*, int, int, int*, int*, int*, int, hipStream_t);
void sm_moe_gemm(const void*, int64_t, int, const int*, const int*, const void*, int, int, void*, int, int, int, int,
                 const float*, hipStream_t);
void sm_bigram_embed(const int64_t*, const void*, float, int64_t, const void*, int64_t, int64_t, int64_t, int*,
                     const int*, const int*, const int*, const int*, int*, float*, void*, int, int, int, hipStream_t);
void sm_post_norm_add(const void*, int64_t, const void*, int64_t, float, float, const float*, const void*, float*, float,
                      const void*, void*, int, int, int, hipStream_t);
int sm_gated_delta_rows(int);
int sm_gated_delta_scan(const void*, int64_t, int, int, int, int, const void*, int64_t, const void*, int64_t, int,
                        const float*, const float*, const void*, int64_t, int, const void*, float, float*, const int*,
                        const int*, const int*, void*, float*, float*, float*, float*, float*, int, int, int,
                        hipStream_t);
void sm_moe_combine(const void*, const int*, const float*, int, int, void*, const void*, int, int, hipStream_t);
}

namespace {

using torch::Tensor;

std::optional<c10::DeviceIndex> dev_of(const Tensor& t) {
  if (t.is_cuda()) return t.get_device();
  return std::nullopt;
}

hipStream_t cur() { return c10::hip::getCurrentHIPStream().stream(); }

bool act_ok(const Tensor& t) { return t.scalar_type() == torch::kBFloat16 || t.scalar_type() == torch::kFloat32; }
int is_f32(const Tensor& t) { return t.scalar_type() == torch::kFloat32 ? 1 : 0; }

#define CHECK_ACT(t, like) \
  TORCH_CHECK((t).is_cuda() && (t).scalar_type() == (like).scalar_type(), #t ": device tensor of the activation type")
#define CHECK_I32(t) TORCH_CHECK((t).is_cuda() && (t).scalar_type() == torch::kInt32 && (t).is_contiguous(), #t ": int32")
#define CHECK_F32(t) TORCH_CHECK((t).is_cuda() && (t).scalar_type() == torch::kFloat32 && (t).is_contiguous(), #t ": fp32")

void check_seq(const Tensor& seq_start, const Tensor& seq_slot, const Tensor& seq_init, int64_t slots) {
  CHECK_I32(seq_start);
  CHECK_I32(seq_slot);
  CHECK_I32(seq_init);
  TORCH_CHECK(seq_start.numel() == seq_slot.numel() + 1 && seq_init.numel() == seq_slot.numel(), "sequence tables");
  (void)slots;
}

void embed_scale(Tensor ids, Tensor table, double scale, Tensor hist) {
  const c10::hip::OptionalHIPGuard g(dev_of(ids));
  TORCH_CHECK(ids.is_cuda() && ids.scalar_type() == torch::kInt64 && ids.is_contiguous(), "ids: int64");
  TORCH_CHECK(table.is_cuda() && act_ok(table) && table.dim() == 2 && table.is_contiguous(), "table");
  CHECK_F32(hist);
  const int T = ids.numel(), d = table.size(1);
  TORCH_CHECK(hist.dim() == 3 && hist.size(0) >= 2 && hist.size(1) == T && hist.size(2) == d, "hist [S, T, d]");
  sm_embed_scale(ids.data_ptr<int64_t>(), table.data_ptr(), (float)scale, hist.data_ptr<float>(),
                 hist.data_ptr<float>() + (int64_t)T * d, T, d, table.size(0), is_f32(table), cur());
}

void zc_norm(Tensor x, Tensor w, double eps, Tensor out) {
  const c10::hip::OptionalHIPGuard g(dev_of(x));
  CHECK_F32(x);
  TORCH_CHECK(x.dim() == 2 && act_ok(w) && w.is_cuda() && w.is_contiguous() && w.numel() == x.size(1), "weight");
  CHECK_ACT(out, w);
  TORCH_CHECK(out.is_contiguous() && out.sizes() == x.sizes(), "out");
  sm_zc_norm(x.data_ptr<float>(), w.data_ptr(), (float)eps, out.data_ptr(), x.size(0), x.size(1), is_f32(w), cur());
}

void add_post_norm(Tensor y, Tensor wp, Tensor ls, Tensor x, double eps, c10::optional<Tensor> wn,
                   c10::optional<Tensor> out) {
  const c10::hip::OptionalHIPGuard g(dev_of(x));
  CHECK_F32(x);
  TORCH_CHECK(x.dim() == 2 && y.dim() == 2 && y.sizes() == x.sizes() && y.stride(1) == 1 && act_ok(y) && y.is_cuda(),
              "y [T, d]");
  const int T = x.size(0), d = x.size(1);
  CHECK_ACT(wp, y);
  CHECK_ACT(ls, y);
  TORCH_CHECK(wp.is_contiguous() && ls.is_contiguous() && wp.numel() == d && ls.numel() == d, "weights");
  const void* wnp = nullptr;
  void* op = nullptr;
  if (wn.has_value()) {
    TORCH_CHECK(out.has_value(), "next norm without output");
    CHECK_ACT(*wn, y);
    CHECK_ACT(*out, y);
    TORCH_CHECK(wn->is_contiguous() && wn->numel() == d && out->is_contiguous() && out->sizes() == x.sizes(), "next");
    wnp = wn->data_ptr();
    op = out->data_ptr();
  }
  sm_add_post_norm(y.data_ptr(), y.stride(0), wp.data_ptr(), ls.data_ptr(), x.data_ptr<float>(), (float)eps, wnp, op, T,
                   d, is_f32(y), cur());
}

void depth_avg_norm(Tensor hist, int64_t n, Tensor coef, int64_t dst, Tensor w, double eps, Tensor out) {
  const c10::hip::OptionalHIPGuard g(dev_of(hist));
  CHECK_F32(hist);
  CHECK_F32(coef);
  TORCH_CHECK(hist.dim() == 3 && n >= 1 && n <= hist.size(0) && dst >= n && dst < hist.size(0) && coef.numel() >= n,
              "depth average: n terms, destination behind them");
  const int T = hist.size(1), d = hist.size(2);
  TORCH_CHECK(w.is_cuda() && act_ok(w) && w.is_contiguous() && w.numel() == d, "weight");
  CHECK_ACT(out, w);
  TORCH_CHECK(out.is_contiguous() && out.dim() == 2 && out.size(0) == T && out.size(1) == d, "out");
  sm_depth_avg_norm(hist.data_ptr<float>(), (int64_t)T * d, n, coef.data_ptr<float>(), dst, w.data_ptr(), (float)eps,
                    out.data_ptr(), T, d, is_f32(w), cur());
}

void xielu(Tensor z, double ap, double aq, Tensor out) {
  const c10::hip::OptionalHIPGuard g(dev_of(z));
  TORCH_CHECK(z.is_cuda() && act_ok(z) && z.is_contiguous(), "z");
  CHECK_ACT(out, z);
  TORCH_CHECK(out.is_contiguous() && out.numel() == z.numel(), "out");
  sm_xielu(z.data_ptr(), (float)ap, (float)aq, out.data_ptr(), z.numel(), is_f32(z), cur());
}

void softcap(Tensor x, double cap) {
  const c10::hip::OptionalHIPGuard g(dev_of(x));
  CHECK_F32(x);
  TORCH_CHECK(cap > 0, "cap");
  sm_softcap(x.data_ptr<float>(), (float)cap, x.numel(), cur());
}

void latent_rope_cache(Tensor q, std::optional<Tensor> kv_, std::optional<Tensor> norm_w_, double eps, Tensor positions,
                       Tensor cos_sin, int64_t H, int64_t dn, int64_t dr, int64_t rot_dims, int64_t R, Tensor slots,
                       Tensor cache, Tensor q_abs, bool interleaved) {
  const c10::hip::OptionalHIPGuard g(dev_of(q));
  TORCH_CHECK(q.is_cuda() && act_ok(q) && q.dim() == 2 && q.stride(1) == 1 && q.size(1) == H * (dn + dr), "q");
  const int T = q.size(0);
  TORCH_CHECK(kv_.has_value() == norm_w_.has_value(), "kv and its norm weight come together");
  if (kv_) {
    const Tensor &kv = *kv_, &norm_w = *norm_w_;
    CHECK_ACT(kv, q);
    TORCH_CHECK(kv.dim() == 2 && kv.stride(1) == 1 && kv.size(0) == T && kv.size(1) == R + dr, "kv");
    CHECK_ACT(norm_w, q);
    TORCH_CHECK(norm_w.is_contiguous() && norm_w.numel() == R, "latent norm weight");
  }
  TORCH_CHECK(positions.is_cuda() && positions.scalar_type() == torch::kInt64 && positions.is_contiguous() &&
                  positions.numel() == T, "positions");
  TORCH_CHECK(slots.is_cuda() && slots.scalar_type() == torch::kInt64 && slots.is_contiguous() && slots.numel() == T,
              "slots");
  CHECK_F32(cos_sin);
  TORCH_CHECK(cos_sin.dim() == 2 && cos_sin.size(1) == rot_dims && rot_dims % 2 == 0 && rot_dims <= dr, "rotary table");
  CHECK_ACT(cache, q);
  TORCH_CHECK(cache.dim() == 3 && cache.is_contiguous() && cache.size(2) == R + dr, "cache [blocks, bs, R + dr]");
  CHECK_ACT(q_abs, q);
  TORCH_CHECK(q_abs.is_contiguous() && q_abs.numel() == (int64_t)T * H * (R + dr), "q_abs");
  // positions and slots are produced by the runner within [0, max_pos) and the pool
  sm_latent_rope_cache(q.data_ptr(), q.stride(0), kv_ ? kv_->data_ptr() : nullptr, kv_ ? kv_->stride(0) : 0,
                       norm_w_ ? norm_w_->data_ptr() : nullptr, (float)eps, positions.data_ptr<int64_t>(),
                       cos_sin.data_ptr<float>(), H, dn, dr, rot_dims, R, slots.data_ptr<int64_t>(), cache.data_ptr(),
                       q_abs.data_ptr(), interleaved ? 1 : 0, T, is_f32(q), cur());
}

void check_head_gate(const std::optional<Tensor>& gate, const Tensor& q_abs) {
  if (!gate) return;
  CHECK_ACT(*gate, q_abs);
  TORCH_CHECK(gate->dim() == 2 && gate->size(0) == q_abs.size(0) && gate->size(1) == q_abs.size(1) &&
                  gate->stride(1) == 1, "gate [T, H]");
}

void latent_attention(Tensor q_abs, Tensor cache, Tensor tables, Tensor row_seq, Tensor row_len, double scale,
                      int64_t R, int64_t qt, Tensor out, std::optional<Tensor> gate) {
  const c10::hip::OptionalHIPGuard g(dev_of(q_abs));
  TORCH_CHECK(q_abs.is_cuda() && act_ok(q_abs) && q_abs.dim() == 3 && q_abs.is_contiguous(), "q_abs [T, H, Dk]");
  const int T = q_abs.size(0), H = q_abs.size(1), Dk = q_abs.size(2);
  CHECK_ACT(cache, q_abs);
  TORCH_CHECK(cache.dim() == 3 && cache.is_contiguous() && cache.size(2) == Dk && R >= 1 && R <= Dk, "cache");
  CHECK_I32(tables);
  CHECK_I32(row_seq);
  CHECK_I32(row_len);
  TORCH_CHECK(tables.dim() == 2 && row_seq.numel() == T && row_len.numel() == T, "row tables");
  CHECK_ACT(out, q_abs);
  TORCH_CHECK(out.is_contiguous() && out.numel() == (int64_t)T * H * R, "out [T, H, R]");
  TORCH_CHECK(qt == 1 || qt == 4, "rows per workgroup: 1 or 4");
  check_head_gate(gate, q_abs);
  const int rc = sm_latent_attention(q_abs.data_ptr(), cache.data_ptr(), tables.data_ptr<int>(), tables.size(1),
                                     cache.size(1), row_seq.data_ptr<int>(), row_len.data_ptr<int>(), (float)scale, H,
                                     R, Dk, T, qt, out.data_ptr(), is_f32(q_abs), gate ? gate->data_ptr() : nullptr,
                                     gate ? gate->stride(0) : 0, cur());
  TORCH_CHECK(rc == 0, "latent_attention: latent rank above 1024 or rows too wide for the LDS tile");
}

bool latent_attention_mfma(Tensor q_abs, Tensor cache, Tensor tables, Tensor items, Tensor row_len, double scale,
                           int64_t R, Tensor out, int64_t nsplit, int64_t split_keys, c10::optional<Tensor> part_o,
                           c10::optional<Tensor> part_ml, std::optional<Tensor> gate) {
  const c10::hip::OptionalHIPGuard g(dev_of(q_abs));
  TORCH_CHECK(q_abs.is_cuda() && q_abs.scalar_type() == torch::kBFloat16 && q_abs.dim() == 3 && q_abs.is_contiguous(),
              "q_abs [T, H, Dk] bf16");
  const int T = q_abs.size(0), H = q_abs.size(1), Dk = q_abs.size(2);
  CHECK_ACT(cache, q_abs);
  TORCH_CHECK(cache.dim() == 3 && cache.is_contiguous() && cache.size(2) == Dk && R >= 1 && R <= Dk, "cache");
  CHECK_I32(tables);
  CHECK_I32(items);
  CHECK_I32(row_len);
  TORCH_CHECK(tables.dim() == 2 && row_len.numel() == T && items.dim() == 2 && items.size(1) == 3, "tables");
  CHECK_ACT(out, q_abs);
  TORCH_CHECK(out.is_contiguous() && out.numel() == (int64_t)T * H * R, "out [T, H, R]");
  // the items are built by ops.seqmix.attention_items from the step's run lengths: rows inside [0, T),
  // tokens * H <= 64
  float *po = nullptr, *pm = nullptr;
  check_head_gate(gate, q_abs);
  TORCH_CHECK(nsplit >= 1 && nsplit <= 1024, "key ranges per item");
  if (nsplit > 1) {
    TORCH_CHECK(split_keys >= 32 && split_keys % 32 == 0, "keys per range: a multiple of 32");
    TORCH_CHECK(part_o.has_value() && part_ml.has_value(), "split step without workspace");
    CHECK_F32(*part_o);
    CHECK_F32(*part_ml);
    TORCH_CHECK(part_o->numel() >= items.size(0) * nsplit * 64 * R && part_ml->numel() >= items.size(0) * nsplit * 128,
                "workspace too small");
    po = part_o->data_ptr<float>();
    pm = part_ml->data_ptr<float>();
  }
  return sm_latent_attention_mfma(q_abs.data_ptr(), cache.data_ptr(), tables.data_ptr<int>(), tables.size(1),
                                  cache.size(1), items.data_ptr<int>(), items.size(0), row_len.data_ptr<int>(),
                                  (float)scale, H, R, Dk, out.data_ptr(), nsplit, split_keys, po, pm,
                                  gate ? gate->data_ptr() : nullptr, gate ? gate->stride(0) : 0, cur()) == 0;
}

void causal_conv_silu(Tensor xz, int64_t C, Tensor w, Tensor b, Tensor state, Tensor seq_start, Tensor seq_slot,
                      Tensor seq_init, int64_t max_q, Tensor out) {
  const c10::hip::OptionalHIPGuard g(dev_of(xz));
  TORCH_CHECK(xz.is_cuda() && act_ok(xz) && xz.dim() == 2 && xz.stride(1) == 1 && xz.size(1) >= C, "xz");
  CHECK_ACT(w, xz);
  CHECK_ACT(b, xz);
  CHECK_ACT(state, xz);
  CHECK_ACT(out, xz);
  TORCH_CHECK(w.dim() == 2 && w.is_contiguous() && w.size(0) == C && b.is_contiguous() && b.numel() == C, "conv weights");
  const int taps = w.size(1);
  TORCH_CHECK(state.dim() == 3 && state.is_contiguous() && state.size(2) == C && state.size(1) >= taps - 1 &&
                  (taps == 1 || state.size(1) == taps - 1), "conv state [slots, taps-1, C]");
  check_seq(seq_start, seq_slot, seq_init, state.size(0));
  TORCH_CHECK(out.is_contiguous() && out.dim() == 2 && out.size(0) == xz.size(0) && out.size(1) == C, "out");
  sm_causal_conv_silu(xz.data_ptr(), xz.stride(0), C, w.data_ptr(), b.data_ptr(), taps, state.data_ptr(),
                      seq_start.data_ptr<int>(), seq_slot.data_ptr<int>(), seq_init.data_ptr<int>(), out.data_ptr(),
                      seq_slot.numel(), max_q, is_f32(xz), cur());
}

void selective_scan(Tensor xc, Tensor dt_raw, Tensor dt_bias, Tensor A, Tensor bc, int64_t R, int64_t N, Tensor D,
                    Tensor xz, int64_t C, Tensor state, Tensor seq_start, Tensor seq_slot, Tensor seq_init, Tensor out) {
  const c10::hip::OptionalHIPGuard g(dev_of(xc));
  TORCH_CHECK(xc.is_cuda() && act_ok(xc) && xc.dim() == 2 && xc.is_contiguous() && xc.size(1) == C, "xc");
  const int T = xc.size(0);
  CHECK_ACT(dt_raw, xc);
  CHECK_ACT(dt_bias, xc);
  CHECK_ACT(bc, xc);
  CHECK_ACT(D, xc);
  CHECK_ACT(xz, xc);
  CHECK_ACT(out, xc);
  CHECK_F32(A);
  CHECK_F32(state);
  TORCH_CHECK(dt_raw.is_contiguous() && dt_raw.sizes() == xc.sizes() && dt_bias.numel() == C && D.numel() == C &&
                  dt_bias.is_contiguous() && D.is_contiguous(), "dt / D");
  TORCH_CHECK(A.dim() == 2 && A.size(0) == C && A.size(1) == N, "A [C, N]");
  TORCH_CHECK(bc.dim() == 2 && bc.stride(1) == 1 && bc.size(0) == T && bc.size(1) >= R + 2 * N, "bc");
  TORCH_CHECK(xz.dim() == 2 && xz.stride(1) == 1 && xz.size(0) == T && xz.size(1) >= 2 * C, "xz");
  TORCH_CHECK(state.dim() == 3 && state.size(1) == C && state.size(2) == N, "state [slots, C, N]");
  check_seq(seq_start, seq_slot, seq_init, state.size(0));
  TORCH_CHECK(out.is_contiguous() && out.sizes() == xc.sizes(), "out");
  const int rc = sm_selective_scan(xc.data_ptr(), dt_raw.data_ptr(), dt_bias.data_ptr(), A.data_ptr<float>(),
                                   bc.data_ptr(), bc.stride(0), R, N, D.data_ptr(), xz.data_ptr(), xz.stride(0), C,
                                   state.data_ptr<float>(), seq_start.data_ptr<int>(), seq_slot.data_ptr<int>(),
                                   seq_init.data_ptr<int>(), out.data_ptr(), seq_slot.numel(), is_f32(xc), cur());
  TORCH_CHECK(rc == 0, "selective_scan: state size above 256");
}

void gdelta_scan(Tensor proj, Tensor wl, Tensor w0, Tensor a_b, Tensor norm_w, double eps, int64_t H, int64_t d,
                 Tensor state, Tensor seq_start, Tensor seq_slot, Tensor seq_init, Tensor out) {
  const c10::hip::OptionalHIPGuard g(dev_of(proj));
  const int64_t HD = H * d;
  TORCH_CHECK(proj.is_cuda() && act_ok(proj) && proj.dim() == 2 && proj.stride(1) == 1 && proj.size(1) >= 5 * HD, "proj");
  const int T = proj.size(0);
  CHECK_ACT(wl, proj);
  CHECK_ACT(w0, proj);
  CHECK_ACT(a_b, proj);
  CHECK_ACT(norm_w, proj);
  CHECK_ACT(out, proj);
  CHECK_F32(state);
  TORCH_CHECK(wl.is_contiguous() && wl.dim() == 2 && wl.size(0) == T && wl.size(1) == HD, "decay logits");
  TORCH_CHECK(w0.is_contiguous() && a_b.is_contiguous() && norm_w.is_contiguous() && w0.numel() == HD &&
                  a_b.numel() == HD && norm_w.numel() == HD, "per-channel vectors");
  TORCH_CHECK(state.dim() == 4 && state.size(1) == H && state.size(2) == d && state.size(3) == d, "state");
  check_seq(seq_start, seq_slot, seq_init, state.size(0));
  TORCH_CHECK(out.is_contiguous() && out.dim() == 2 && out.size(0) == T && out.size(1) == HD, "out");
  const int rc = sm_gdelta_scan(proj.data_ptr(), proj.stride(0), wl.data_ptr(), w0.data_ptr(), a_b.data_ptr(),
                                norm_w.data_ptr(), (float)eps, H, d, state.data_ptr<float>(),
                                seq_start.data_ptr<int>(), seq_slot.data_ptr<int>(), seq_init.data_ptr<int>(),
                                out.data_ptr(), seq_slot.numel(), is_f32(proj), cur());
  TORCH_CHECK(rc == 0, "gdelta_scan: head size above 256");
}

void hyper_embed(Tensor ids, Tensor table, Tensor X) {
  const c10::hip::OptionalHIPGuard g(dev_of(ids));
  TORCH_CHECK(ids.is_cuda() && ids.scalar_type() == torch::kInt64 && ids.is_contiguous(), "ids: int64");
  TORCH_CHECK(table.is_cuda() && act_ok(table) && table.dim() == 2 && table.is_contiguous(), "table");
  CHECK_F32(X);
  const int T = ids.numel(), d = table.size(1);
  TORCH_CHECK(X.dim() == 3 && X.size(0) >= 1 && X.size(0) <= 16 && X.size(1) == T && X.size(2) == d, "X [S <= 16, T, d]");
  sm_hyper_embed(ids.data_ptr<int64_t>(), table.data_ptr(), table.size(0), X.data_ptr<float>(), X.size(0), T, d,
                 is_f32(table), cur());
}

void check_streams(const Tensor& X) {
  CHECK_F32(X);
  TORCH_CHECK(X.dim() == 3 && X.size(0) >= 1 && X.size(0) <= 16 && X.size(2) <= 16384, "X [S <= 16, T, d <= 16384]");
}

void hyper_norm(Tensor X, Tensor w_in, Tensor norm_w, double eps, Tensor out) {
  const c10::hip::OptionalHIPGuard g(dev_of(X));
  check_streams(X);
  CHECK_F32(w_in);
  const int S = X.size(0), T = X.size(1), d = X.size(2);
  TORCH_CHECK(w_in.numel() == S && norm_w.is_cuda() && act_ok(norm_w) && norm_w.is_contiguous() && norm_w.numel() == d,
              "weights");
  CHECK_ACT(out, norm_w);
  TORCH_CHECK(out.is_contiguous() && out.dim() == 2 && out.size(0) == T && out.size(1) == d, "out [T, d]");
  sm_hyper_norm(X.data_ptr<float>(), w_in.data_ptr<float>(), norm_w.data_ptr(), (float)eps, out.data_ptr(), S, T, d,
                is_f32(norm_w), cur());
}

void hyper_update_norm(Tensor X, Tensor y, Tensor mix, Tensor w_out, std::optional<Tensor> next_in,
                       std::optional<Tensor> next_w, double eps, std::optional<Tensor> out) {
  const c10::hip::OptionalHIPGuard g(dev_of(X));
  check_streams(X);
  CHECK_F32(mix);
  CHECK_F32(w_out);
  const int S = X.size(0), T = X.size(1), d = X.size(2);
  TORCH_CHECK(y.is_cuda() && act_ok(y) && y.dim() == 2 && y.size(0) == T && y.size(1) == d && y.stride(1) == 1, "y [T, d]");
  TORCH_CHECK(mix.numel() == (int64_t)S * S && w_out.numel() == S, "mix [S, S], out [S]");
  const float* nin = nullptr;
  const void* nw = nullptr;
  void* o = nullptr;
  if (next_w) {
    TORCH_CHECK(next_in && out, "next_in and out come with next_w");
    CHECK_F32(*next_in);
    CHECK_ACT(*next_w, y);
    CHECK_ACT(*out, y);
    TORCH_CHECK(next_in->numel() == S && next_w->is_contiguous() && next_w->numel() == d && out->is_contiguous() &&
                    out->dim() == 2 && out->size(0) == T && out->size(1) == d, "next norm shapes");
    nin = next_in->data_ptr<float>();
    nw = next_w->data_ptr();
    o = out->data_ptr();
  }
  sm_hyper_update_norm(X.data_ptr<float>(), y.data_ptr(), y.stride(0), mix.data_ptr<float>(), w_out.data_ptr<float>(),
                       nin, nw, (float)eps, o, S, T, d, is_f32(y), cur());
}

void gated_act(Tensor gu, int64_t F, int64_t kind, Tensor out) {
  const c10::hip::OptionalHIPGuard g(dev_of(gu));
  TORCH_CHECK(gu.is_cuda() && act_ok(gu) && gu.dim() == 2 && gu.stride(1) == 1 && gu.size(1) >= 2 * F && F >= 1, "gu");
  CHECK_ACT(out, gu);
  TORCH_CHECK(out.is_contiguous() && out.dim() == 2 && out.size(0) == gu.size(0) && out.size(1) == F &&
                  (kind == 0 || kind == 1), "out [T, F]");
  sm_gated_act(gu.data_ptr(), gu.stride(0), F, kind, out.data_ptr(), gu.size(0), is_f32(gu), cur());
}

void qkv_rope_cache(Tensor qkv, std::optional<Tensor> bias, Tensor positions, std::optional<Tensor> cos_sin, int64_t Hq,
                    int64_t Hkv, int64_t dim, int64_t vdim, int64_t rot_dims, bool interleaved, bool unit, double eps,
                    std::optional<Tensor> v_first, int64_t v_mode, double lam, Tensor slots, Tensor cache,
                    Tensor q_out, std::optional<Tensor> qk_w, bool norm_first, bool v_from_k) {
  const c10::hip::OptionalHIPGuard g(dev_of(qkv));
  TORCH_CHECK(qkv.is_cuda() && act_ok(qkv) && qkv.dim() == 2 && qkv.stride(1) == 1, "qkv");
  TORCH_CHECK(!v_from_k || (vdim == dim && v_mode == 0), "keys as values: vdim == dim, no value mixing");
  const int64_t T = qkv.size(0), n = (Hq + Hkv) * dim + (v_from_k ? 0 : Hkv * vdim);
  TORCH_CHECK(Hq >= 1 && Hkv >= 1 && Hq % Hkv == 0 && dim >= 1 && dim <= 512 && vdim >= 1 && qkv.size(1) >= n, "sizes");
  TORCH_CHECK(rot_dims >= 0 && rot_dims <= dim && rot_dims % 2 == 0, "rotary dims");
  TORCH_CHECK(positions.is_cuda() && positions.scalar_type() == torch::kInt64 && positions.is_contiguous() &&
                  positions.numel() == T && slots.is_cuda() && slots.scalar_type() == torch::kInt64 &&
                  slots.is_contiguous() && slots.numel() == T, "positions / slots: int64 [T]");
  if (bias) {
    CHECK_F32(*bias);
    TORCH_CHECK(bias->numel() == n, "bias over q | k | v");
  }
  if (rot_dims) {
    TORCH_CHECK(cos_sin.has_value(), "cos_sin");
    CHECK_F32(*cos_sin);
    TORCH_CHECK(cos_sin->dim() == 2 && cos_sin->size(1) == rot_dims, "cos_sin [max_pos, rot_dims]");
  }
  if (qk_w) {
    CHECK_F32(*qk_w);
    TORCH_CHECK(unit && qk_w->numel() == 2 * dim, "qk_w [2, dim] goes with the unit norm");
  }
  TORCH_CHECK(v_mode >= 0 && v_mode <= 2, "v_mode");
  if (v_mode) {
    TORCH_CHECK(v_first.has_value(), "v_first");
    CHECK_F32(*v_first);
    TORCH_CHECK(v_first->numel() == T * Hkv * vdim, "v_first [T, Hkv * vdim]");
  }
  CHECK_ACT(cache, qkv);
  CHECK_ACT(q_out, qkv);
  TORCH_CHECK(cache.dim() == 4 && cache.is_contiguous() && cache.size(1) == Hkv && cache.size(3) == dim + vdim,
              "cache [blocks, Hkv, bs, dim + vdim]");
  TORCH_CHECK(q_out.is_contiguous() && q_out.numel() == T * Hq * dim, "q_out [T, Hq, dim]");
  sm_qkv_rope_cache(qkv.data_ptr(), qkv.stride(0), bias ? bias->data_ptr<float>() : nullptr,
                    positions.data_ptr<int64_t>(), rot_dims ? cos_sin->data_ptr<float>() : nullptr, Hq, Hkv, dim, vdim,
                    rot_dims, interleaved ? 1 : 0, unit ? 1 : 0, (float)eps, v_mode ? v_first->data_ptr<float>() : nullptr,
                    v_mode, (float)lam, slots.data_ptr<int64_t>(), cache.data_ptr(), cache.size(2), q_out.data_ptr(),
                    qk_w ? qk_w->data_ptr<float>() : nullptr, norm_first ? 1 : 0, v_from_k ? 1 : 0, T, is_f32(qkv),
                    cur());
}

void check_gqa(const Tensor& q, const Tensor& cache, int64_t dim, int64_t vdim, const Tensor& tables,
               const Tensor& row_len, const std::optional<Tensor>& gate, const Tensor& out,
               const std::optional<Tensor>& slopes, int64_t chunk, const std::optional<Tensor>& sinks) {
  TORCH_CHECK(chunk >= 0 && chunk < (1ll << 30), "chunk");
  for (const auto* v : {&slopes, &sinks})
    if (*v) {
      CHECK_F32(**v);
      TORCH_CHECK((*v)->numel() == q.size(1), "slopes / sinks: fp32 [Hq]");
    }
  TORCH_CHECK(q.is_cuda() && act_ok(q) && q.dim() == 3 && q.is_contiguous() && q.size(2) == dim, "q [T, Hq, dim]");
  CHECK_ACT(cache, q);
  CHECK_ACT(out, q);
  TORCH_CHECK(cache.dim() == 4 && cache.is_contiguous() && cache.size(3) == dim + vdim && q.size(1) % cache.size(1) == 0,
              "cache [blocks, Hkv, bs, dim + vdim]");
  CHECK_I32(tables);
  CHECK_I32(row_len);
  TORCH_CHECK(tables.dim() == 2 && row_len.numel() == q.size(0), "tables [n, W], row_len [T]");
  TORCH_CHECK(out.is_contiguous() && out.numel() == q.size(0) * q.size(1) * vdim, "out [T, Hq * vdim]");
  if (gate) {
    CHECK_ACT(*gate, q);
    TORCH_CHECK(gate->dim() == 2 && gate->size(0) == q.size(0) && gate->size(1) == q.size(1) * vdim &&
                    gate->stride(1) == 1, "gate [T, Hq * vdim]");
  }
}

void check_window(int64_t window, int64_t keep, int64_t chunk) {
  TORCH_CHECK(window >= 0 && window < (1ll << 30) && keep >= 0 && keep < (1ll << 30) && (window == 0 || chunk == 0),
              "window / kept first tokens (not with chunks)");
}

void grouped_attention(Tensor q, Tensor cache, int64_t dim, int64_t vdim, Tensor tables, Tensor row_seq, Tensor row_len,
                       double scale, std::optional<Tensor> gate, int64_t rows_per_group, Tensor out,
                       std::optional<Tensor> slopes, int64_t chunk, std::optional<Tensor> sinks, int64_t window,
                       int64_t keep) {
  const c10::hip::OptionalHIPGuard g(dev_of(q));
  check_gqa(q, cache, dim, vdim, tables, row_len, gate, out, slopes, chunk, sinks);
  check_window(window, keep, chunk);
  CHECK_I32(row_seq);
  TORCH_CHECK(row_seq.numel() == q.size(0) && (rows_per_group == 1 || rows_per_group == 4), "row_seq [T]");
  const int rc = sm_grouped_attention(q.data_ptr(), cache.data_ptr(), tables.data_ptr<int>(), tables.size(1),
                                      cache.size(2), row_seq.data_ptr<int>(), row_len.data_ptr<int>(), (float)scale,
                                      q.size(1), cache.size(1), dim, vdim, q.size(0), rows_per_group,
                                      gate ? gate->data_ptr() : nullptr, gate ? gate->stride(0) : 0, out.data_ptr(),
                                      is_f32(q), slopes ? slopes->data_ptr<float>() : nullptr, chunk,
                                      sinks ? sinks->data_ptr<float>() : nullptr, window, keep, cur());
  TORCH_CHECK(rc == 0, "grouped_attention: head sizes too large for the kernel (vdim <= 1024, one key tile in LDS)");
}

bool grouped_attention_mfma(Tensor q, Tensor cache, int64_t dim, int64_t vdim, Tensor tables, Tensor items,
                            Tensor row_len, double scale, std::optional<Tensor> gate, Tensor out, int64_t nsplit,
                            int64_t split_keys, std::optional<Tensor> part_o, std::optional<Tensor> part_ml,
                            int64_t rb, std::optional<Tensor> slopes, int64_t chunk, std::optional<Tensor> sinks,
                            int64_t window, int64_t keep) {
  const c10::hip::OptionalHIPGuard g(dev_of(q));
  check_gqa(q, cache, dim, vdim, tables, row_len, gate, out, slopes, chunk, sinks);
  check_window(window, keep, chunk);
  TORCH_CHECK(q.scalar_type() == torch::kBFloat16, "bf16 only");
  CHECK_I32(items);
  TORCH_CHECK(items.dim() == 2 && items.size(1) == 3, "items [n, 3]");
  const int64_t n = items.size(0), Hkv = cache.size(1);
  float *po = nullptr, *pm = nullptr;
  TORCH_CHECK(nsplit >= 1 && (rb == 1 || rb == 2) && (nsplit == 1 || rb == 1), "nsplit / rows per wave");
  if (nsplit > 1) {
    TORCH_CHECK(part_o && part_ml && split_keys > 0 && split_keys % 32 == 0, "split workspace");
    CHECK_F32(*part_o);
    CHECK_F32(*part_ml);
    TORCH_CHECK(part_o->numel() >= n * Hkv * nsplit * 64 * vdim && part_ml->numel() >= n * Hkv * nsplit * 128,
                "split workspace too small");
    po = part_o->data_ptr<float>();
    pm = part_ml->data_ptr<float>();
  }
  const int rc = sm_grouped_attention_mfma(q.data_ptr(), cache.data_ptr(), tables.data_ptr<int>(), tables.size(1),
                                           cache.size(2), items.data_ptr<int>(), n, row_len.data_ptr<int>(),
                                           (float)scale, q.size(1), Hkv, dim, vdim, gate ? gate->data_ptr() : nullptr,
                                           gate ? gate->stride(0) : 0, out.data_ptr(), nsplit, split_keys, po, pm,
                                           rb, slopes ? slopes->data_ptr<float>() : nullptr, chunk,
                                           sinks ? sinks->data_ptr<float>() : nullptr, window, keep, cur());
  return rc == 0;
}

void moe_route_scores(Tensor logits, Tensor correction, int64_t k, Tensor ids, Tensor w) {
  const c10::hip::OptionalHIPGuard g(dev_of(logits));
  CHECK_F32(logits);
  CHECK_F32(correction);
  CHECK_I32(ids);
  CHECK_F32(w);
  const int T = logits.size(0), E = logits.size(1);
  TORCH_CHECK(logits.dim() == 2 && k >= 1 && k <= E && correction.numel() == E && ids.numel() == (int64_t)T * k &&
                  w.numel() == (int64_t)T * k, "router shapes");
  sm_moe_route_scores(logits.data_ptr<float>(), correction.data_ptr<float>(), E, k, ids.data_ptr<int>(),
                      w.data_ptr<float>(), T, cur());
}

void moe_route(Tensor logits, int64_t k, Tensor ids, Tensor w, bool sigmoid) {
  const c10::hip::OptionalHIPGuard g(dev_of(logits));
  CHECK_F32(logits);
  CHECK_I32(ids);
  CHECK_F32(w);
  const int T = logits.size(0), E = logits.size(1);
  TORCH_CHECK(logits.dim() == 2 && k >= 1 && k <= E && ids.numel() == (int64_t)T * k && w.numel() == (int64_t)T * k,
              "router shapes");
  sm_moe_route(logits.data_ptr<float>(), E, k, ids.data_ptr<int>(), w.data_ptr<float>(), T, sigmoid ? 1 : 0, cur());
}

void moe_group(Tensor ids, int64_t E, Tensor slot_row, Tensor tile_e, Tensor pair_slot) {
  const c10::hip::OptionalHIPGuard g(dev_of(ids));
  CHECK_I32(ids);
  CHECK_I32(slot_row);
  CHECK_I32(tile_e);
  CHECK_I32(pair_slot);
  const int64_t n = ids.numel(), mt = tile_e.numel();
  TORCH_CHECK(slot_row.numel() == mt * 64 && pair_slot.numel() == n && mt * 64 >= n + E * 63 && E <= 8192,
              "tile tables too small for n pairs over E experts");
  sm_moe_group(ids.data_ptr<int>(), n, E, slot_row.data_ptr<int>(), tile_e.data_ptr<int>(), pair_slot.data_ptr<int>(),
               mt, cur());
}

void moe_gemm(Tensor A, int64_t kdiv, Tensor slot_row, Tensor tile_e, Tensor W, Tensor C, int64_t act, int64_t rows,
              std::optional<Tensor> row_w) {
  const c10::hip::OptionalHIPGuard g(dev_of(A));
  TORCH_CHECK(A.is_cuda() && act_ok(A) && A.dim() == 2 && A.stride(1) == 1, "A");
  CHECK_ACT(W, A);
  CHECK_ACT(C, A);
  CHECK_I32(slot_row);
  CHECK_I32(tile_e);
  TORCH_CHECK(W.dim() == 3 && W.is_contiguous() && W.size(2) == A.size(1), "W [E, N, K]");
  const int64_t mt = tile_e.numel();
  TORCH_CHECK(act >= 0 && act <= 3 && (act < 2 || W.size(1) % 2 == 0), "epilogue");
  const int64_t N = act >= 2 ? W.size(1) / 2 : W.size(1);  // gated: W holds [gate rows | up rows]
  TORCH_CHECK(slot_row.numel() == mt * 64 && C.is_contiguous() && C.dim() == 2 && C.size(0) == mt * 64 &&
                  C.size(1) == N, "C [tiles * 64, N]");
  TORCH_CHECK(kdiv > 0 || A.size(0) == mt * 64, "A rows are the tile slots");
  if (row_w) {  // indexed by the pair numbers in slot_row: one weight per (token, choice)
    CHECK_F32(*row_w);
    TORCH_CHECK(act >= 2 && kdiv > 0 && row_w->numel() == A.size(0) * kdiv, "row_w [T, k] with a gated epilogue");
  }
  sm_moe_gemm(A.data_ptr(), A.stride(0), kdiv, slot_row.data_ptr<int>(), tile_e.data_ptr<int>(), W.data_ptr(),
              N, W.size(2), C.data_ptr(), mt, rows, (int)act, is_f32(A), row_w ? row_w->data_ptr<float>() : nullptr,
              cur());
}

void moe_combine(Tensor y, Tensor pair_slot, std::optional<Tensor> w, Tensor out, std::optional<Tensor> h) {
  const c10::hip::OptionalHIPGuard g(dev_of(y));
  TORCH_CHECK(y.is_cuda() && act_ok(y) && y.dim() == 2 && y.is_contiguous(), "y");
  CHECK_I32(pair_slot);
  CHECK_ACT(out, y);
  TORCH_CHECK(out.dim() == 2, "out [T, d]");
  if (out.size(0) == 0) return;
  const int T = out.size(0), d = out.size(1);
  TORCH_CHECK(out.is_contiguous() && y.size(1) == d && pair_slot.numel() % T == 0 && pair_slot.numel() >= T,
              "combine shapes");
  const int k = pair_slot.numel() / T;
  if (w) {  // without weights the rows are added as they are
    CHECK_F32(*w);
    TORCH_CHECK(w->dim() == 2 && w->size(0) == T && pair_slot.numel() == w->numel(), "w [T, k]");
  }
  // h: the tokens' inputs, read for pairs marked -1 (identity experts); without it no pair may be -1
  if (h) {
    CHECK_ACT(*h, y);
    TORCH_CHECK(h->dim() == 2 && h->is_contiguous() && h->size(0) == T && h->size(1) == d, "h [T, d]");
  }
  sm_moe_combine(y.data_ptr(), pair_slot.data_ptr<int>(), w ? w->data_ptr<float>() : nullptr, k, d, out.data_ptr(),
                 h ? h->data_ptr() : y.data_ptr(), T, is_f32(y), cur());
}

void bigram_embed(Tensor ids, Tensor table, double scale, std::optional<Tensor> bigram, int64_t buckets,
                  int64_t mul_prev, int64_t mul_cur, Tensor prev_state, Tensor row_seq, Tensor seq_start,
                  Tensor seq_slot, Tensor seq_init, Tensor x, Tensor out) {
  const c10::hip::OptionalHIPGuard g(dev_of(ids));
  TORCH_CHECK(ids.is_cuda() && ids.scalar_type() == torch::kInt64 && ids.is_contiguous(), "ids: int64");
  TORCH_CHECK(table.is_cuda() && act_ok(table) && table.dim() == 2 && table.is_contiguous(), "table");
  const int T = ids.numel(), d = table.size(1);
  CHECK_F32(x);
  CHECK_ACT(out, table);
  TORCH_CHECK(x.dim() == 2 && x.size(0) == T && x.size(1) == d && out.is_contiguous() && out.sizes() == x.sizes(),
              "x, out [T, d]");
  CHECK_I32(prev_state);
  CHECK_I32(row_seq);
  check_seq(seq_start, seq_slot, seq_init, prev_state.numel());
  TORCH_CHECK(row_seq.numel() == T, "row_seq [T]");
  Tensor rows;
  if (bigram) {
    CHECK_ACT(*bigram, table);
    TORCH_CHECK(buckets >= 1 && bigram->dim() == 2 && bigram->is_contiguous() && bigram->size(0) == buckets + 1 &&
                    bigram->size(1) == d, "bigram [buckets + 1, d]");
    rows = torch::empty({T}, torch::dtype(torch::kInt32).device(ids.device()));
  }
  sm_bigram_embed(ids.data_ptr<int64_t>(), table.data_ptr(), (float)scale, table.size(0),
                  bigram ? bigram->data_ptr() : nullptr, buckets, mul_prev, mul_cur, prev_state.data_ptr<int>(),
                  row_seq.data_ptr<int>(), seq_start.data_ptr<int>(), seq_slot.data_ptr<int>(),
                  seq_init.data_ptr<int>(), bigram ? rows.data_ptr<int>() : nullptr, x.data_ptr<float>(),
                  out.data_ptr(), T, d, is_f32(table), cur());
}

void post_norm_add(Tensor y, std::optional<Tensor> y2, double a, double b, std::optional<Tensor> bias, Tensor w_post,
                   Tensor x, double eps, std::optional<Tensor> next_w, Tensor out) {
  const c10::hip::OptionalHIPGuard g(dev_of(y));
  TORCH_CHECK(y.is_cuda() && act_ok(y) && y.dim() == 2 && y.stride(1) == 1, "y");
  const int T = y.size(0), d = y.size(1);
  CHECK_F32(x);
  CHECK_ACT(w_post, y);
  CHECK_ACT(out, y);
  TORCH_CHECK(x.dim() == 2 && x.size(0) == T && x.size(1) == d && d <= 65536 && w_post.is_contiguous() &&
                  w_post.numel() == d && out.is_contiguous() && out.sizes() == x.sizes(), "x, out [T, d]; w [d]");
  if (y2) {
    CHECK_ACT(*y2, y);
    TORCH_CHECK(y2->dim() == 2 && y2->stride(1) == 1 && y2->size(0) == T && y2->size(1) == d, "y2 [T, d]");
  }
  if (bias) {
    CHECK_F32(*bias);
    TORCH_CHECK(bias->numel() == d, "bias [d]");
  }
  if (next_w) {
    CHECK_ACT(*next_w, y);
    TORCH_CHECK(next_w->is_contiguous() && next_w->numel() == d, "next_w [d]");
  }
  sm_post_norm_add(y.data_ptr(), y.stride(0), y2 ? y2->data_ptr() : nullptr, y2 ? y2->stride(0) : 0, (float)a,
                   (float)b, bias ? bias->data_ptr<float>() : nullptr, w_post.data_ptr(), x.data_ptr<float>(),
                   (float)eps, next_w ? next_w->data_ptr() : nullptr, out.data_ptr(), T, d, is_f32(y), cur());
}

void gated_delta_scan(Tensor xc, int64_t G, int64_t dk, int64_t H, int64_t dv, Tensor beta_raw, Tensor decay_raw,
                      Tensor A, Tensor dt_bias, Tensor gate_raw, bool gate_sigmoid, Tensor norm_w, double eps,
                      Tensor state, Tensor seq_start, Tensor seq_slot, Tensor seq_init, Tensor out) {
  const c10::hip::OptionalHIPGuard g(dev_of(xc));
  TORCH_CHECK(G >= 1 && H >= 1 && H % G == 0 && dk >= 1 && dv >= 1, "head counts and sizes");
  TORCH_CHECK(xc.is_cuda() && act_ok(xc) && xc.dim() == 2 && xc.stride(1) == 1 && xc.size(1) >= 2 * G * dk + H * dv,
              "xc [T, q | k | v]");
  const int64_t T = xc.size(0);
  CHECK_ACT(beta_raw, xc);
  CHECK_ACT(decay_raw, xc);
  CHECK_ACT(gate_raw, xc);
  CHECK_ACT(norm_w, xc);
  CHECK_ACT(out, xc);
  CHECK_F32(A);
  CHECK_F32(dt_bias);
  CHECK_F32(state);
  for (const Tensor* t : {&beta_raw, &decay_raw, &gate_raw})
    TORCH_CHECK(t->dim() == 2 && t->size(0) == T && t->stride(1) == 1, "beta / decay / gate: [T, n] rows");
  const bool per_channel = decay_raw.size(1) == H * dk && dk > 1;
  TORCH_CHECK(beta_raw.size(1) == H && gate_raw.size(1) == H * dv && (per_channel || decay_raw.size(1) == H),
              "beta [T, H], decay [T, H] or [T, H dk], gate [T, H dv]");
  TORCH_CHECK(A.numel() == H && dt_bias.numel() == decay_raw.size(1) && norm_w.is_contiguous() && norm_w.numel() == dv,
              "A [H], dt_bias like the decay, norm_w [dv]");
  TORCH_CHECK(state.dim() == 4 && state.size(1) == H && state.size(2) == dk && state.size(3) == dv,
              "state [slots, H, dk, dv]");
  check_seq(seq_start, seq_slot, seq_init, state.size(0));
  TORCH_CHECK(out.is_contiguous() && out.dim() == 2 && out.size(0) == T && out.size(1) == H * dv, "out [T, H dv]");
  const int64_t KD = sm_gated_delta_rows(dk);
  TORCH_CHECK(KD > 0, "gated_delta_scan: key size above 256");
  TORCH_CHECK(seq_slot.numel() <= 65535, "too many sequences in a step");
  // fp32 workspaces of the three kernels: [qn | kn | dec | beta | o_raw]
  const int64_t n_qk = T * G * KD, n_dec = per_channel ? T * H * KD : T * H, n_b = T * H, n_o = T * H * dv;
  Tensor ws = torch::empty({2 * n_qk + n_dec + n_b + n_o + 4}, torch::dtype(torch::kFloat32).device(xc.device()));
  float* w0 = ws.data_ptr<float>();
  const int rc = sm_gated_delta_scan(
      xc.data_ptr(), xc.stride(0), G, dk, H, dv, beta_raw.data_ptr(), beta_raw.stride(0), decay_raw.data_ptr(),
      decay_raw.stride(0), per_channel ? 1 : 0, A.data_ptr<float>(), dt_bias.data_ptr<float>(), gate_raw.data_ptr(),
      gate_raw.stride(0), gate_sigmoid ? 1 : 0, norm_w.data_ptr(), (float)eps, state.data_ptr<float>(),
      seq_start.data_ptr<int>(), seq_slot.data_ptr<int>(), seq_init.data_ptr<int>(), out.data_ptr(), w0, w0 + n_qk,
      w0 + 2 * n_qk, w0 + 2 * n_qk + n_dec, w0 + 2 * n_qk + n_dec + n_b, T, seq_slot.numel(), is_f32(xc), cur());
  TORCH_CHECK(rc == 0, "gated_delta_scan: key size above 256");
}

void embed_norm(Tensor ids, Tensor table, Tensor w, double eps, Tensor x, Tensor out) {
  const c10::hip::OptionalHIPGuard g(dev_of(x));
  TORCH_CHECK(ids.is_cuda() && ids.scalar_type() == torch::kInt64 && ids.is_contiguous() && ids.dim() == 1, "ids");
  TORCH_CHECK(table.is_cuda() && act_ok(table) && table.dim() == 2 && table.is_contiguous(), "table");
  const int64_t T = ids.numel(), d = table.size(1);
  CHECK_ACT(w, table);
  CHECK_ACT(out, table);
  CHECK_F32(x);
  TORCH_CHECK(w.is_contiguous() && w.numel() == d && x.numel() == T * d && out.is_contiguous() && out.numel() == T * d,
              "w [d], x / out [T, d]");
  sm_embed_norm(ids.data_ptr<int64_t>(), table.data_ptr(), table.size(0), w.data_ptr(), (float)eps,
                x.data_ptr<float>(), out.data_ptr(), T, d, is_f32(table), cur());
}

void rms_norm(Tensor y, Tensor w, double eps, Tensor out) {
  const c10::hip::OptionalHIPGuard g(dev_of(y));
  TORCH_CHECK(y.is_cuda() && act_ok(y) && y.dim() == 2 && y.stride(1) == 1, "y [T, n] rows");
  CHECK_ACT(w, y);
  CHECK_ACT(out, y);
  TORCH_CHECK(w.is_contiguous() && w.numel() == y.size(1) && out.is_contiguous() && out.numel() == y.numel(),
              "w [n], out [T, n]");
  sm_rms_norm_rows(y.data_ptr(), y.stride(0), w.data_ptr(), (float)eps, out.data_ptr(), y.size(0), y.size(1),
                   is_f32(y), cur());
}

void relu2(Tensor z, Tensor out) {
  const c10::hip::OptionalHIPGuard g(dev_of(z));
  TORCH_CHECK(z.is_cuda() && act_ok(z) && z.is_contiguous(), "z");
  CHECK_ACT(out, z);
  TORCH_CHECK(out.is_contiguous() && out.numel() == z.numel(), "out");
  sm_relu2(z.data_ptr(), out.data_ptr(), z.numel(), is_f32(z), cur());
}

void input_conv(Tensor h, Tensor w, Tensor state, Tensor row_seq, Tensor seq_start, Tensor seq_slot, Tensor seq_init,
                int64_t max_q, Tensor out) {
  const c10::hip::OptionalHIPGuard g(dev_of(h));
  TORCH_CHECK(h.is_cuda() && act_ok(h) && h.dim() == 2 && h.is_contiguous(), "h [T, C]");
  const int64_t T = h.size(0), C = h.size(1);
  CHECK_ACT(w, h);
  CHECK_ACT(state, h);
  CHECK_ACT(out, h);
  TORCH_CHECK(w.dim() == 2 && w.is_contiguous() && w.size(0) == C && w.size(1) >= 1, "conv weights [C, taps]");
  const int taps = w.size(1);
  TORCH_CHECK(state.dim() == 3 && state.is_contiguous() && state.size(2) == C &&
                  (taps == 1 || state.size(1) == taps - 1), "conv state [slots, taps-1, C]");
  check_seq(seq_start, seq_slot, seq_init, state.size(0));
  CHECK_I32(row_seq);
  TORCH_CHECK(row_seq.numel() == T && seq_slot.numel() <= 65535 && max_q >= 1 && max_q <= T, "row_seq [T], longest run");
  TORCH_CHECK(out.is_contiguous() && out.numel() == T * C, "out [T, C]");
  sm_input_conv(h.data_ptr(), C, w.data_ptr(), taps, state.data_ptr(), row_seq.data_ptr<int>(),
                seq_start.data_ptr<int>(), seq_slot.data_ptr<int>(), seq_init.data_ptr<int>(), out.data_ptr(), T,
                seq_slot.numel(), max_q, is_f32(h), cur());
}

// chunks: int32 [4 nc + 1 + nseq + 1] = [chunk bounds (nc + 1) | 0 .. nc - 1 | nc zeros | nc ones | each
// sequence's first chunk (nseq + 1)], built by the caller from the step's run lengths; absent: token by token.
void hgrn2_scan(Tensor p, int64_t H, int64_t dk, int64_t dv, Tensor f_bias, Tensor lower, Tensor norm_w, double eps,
                Tensor state, Tensor seq_start, Tensor seq_slot, Tensor seq_init, Tensor out,
                std::optional<Tensor> chunks, int64_t nc) {
  const c10::hip::OptionalHIPGuard g(dev_of(p));
  TORCH_CHECK(H >= 1 && dk >= 1 && dv >= 1, "head count and sizes");
  TORCH_CHECK(p.is_cuda() && act_ok(p) && p.dim() == 2 && p.stride(1) == 1 && p.size(1) >= 2 * H * dk + H * dv,
              "p [T, q | f | v]");
  const int64_t T = p.size(0);
  CHECK_ACT(norm_w, p);
  CHECK_ACT(out, p);
  CHECK_F32(f_bias);
  CHECK_F32(lower);
  CHECK_F32(state);
  TORCH_CHECK(f_bias.numel() == H * dk && lower.numel() == H * dk && norm_w.is_contiguous() && norm_w.numel() == dv,
              "f_bias, lower [H dk], norm_w [dv]");
  TORCH_CHECK(state.dim() == 4 && state.size(1) == H && state.size(2) == dk && state.size(3) == dv,
              "state [slots, H, dk, dv]");
  check_seq(seq_start, seq_slot, seq_init, state.size(0));
  TORCH_CHECK(out.is_contiguous() && out.dim() == 2 && out.size(0) == T && out.size(1) == H * dv, "out [T, H dv]");
  const int64_t KD = sm_gated_delta_rows(dk);
  TORCH_CHECK(KD > 0, "hgrn2_scan: key size above 256");
  TORCH_CHECK(seq_slot.numel() <= 65535, "too many sequences in a step");
  // fp32 workspaces of the three kernels: [qn | kn | dec | o_raw]
  const int64_t n_qk = T * H * KD, n_o = T * H * dv;
  const int64_t nseq = seq_slot.numel();
  const int* ch = nullptr;
  int64_t n_cs = 0, n_cd = 0;
  if (chunks) {
    CHECK_I32(*chunks);
    TORCH_CHECK(nc >= 1 && nc <= 65535 && chunks->numel() == 4 * nc + 1 + nseq + 1, "chunk table");
    ch = chunks->data_ptr<int>();
    n_cs = nc * H * dk * dv;
    n_cd = nc * H * KD;
  } else {
    nc = 0;
  }
  Tensor ws = torch::empty({3 * n_qk + n_o + n_cs + n_cd + 4}, torch::dtype(torch::kFloat32).device(p.device()));
  float* w0 = ws.data_ptr<float>();
  float* wc = w0 + 3 * n_qk + n_o;
  const int rc = sm_hgrn2_scan(p.data_ptr(), p.stride(0), H, dk, dv, f_bias.data_ptr<float>(), lower.data_ptr<float>(),
                               norm_w.data_ptr(), (float)eps, state.data_ptr<float>(), seq_start.data_ptr<int>(),
                               seq_slot.data_ptr<int>(), seq_init.data_ptr<int>(), out.data_ptr(), w0, w0 + n_qk,
                               w0 + 2 * n_qk, w0 + 3 * n_qk, T, nseq, is_f32(p), nc, ch, ch ? ch + nc + 1 : nullptr,
                               ch ? ch + 2 * nc + 1 : nullptr, ch ? ch + 3 * nc + 1 : nullptr,
                               ch ? ch + 4 * nc + 1 : nullptr, wc, wc + n_cs, cur());
  TORCH_CHECK(rc == 0, "hgrn2_scan: key size above 256");
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.def("embed_scale", &embed_scale);
  m.def("zc_norm", &zc_norm);
  m.def("add_post_norm", &add_post_norm);
  m.def("depth_avg_norm", &depth_avg_norm);
  m.def("xielu", &xielu);
  m.def("softcap", &softcap);
  m.def("latent_rope_cache", &latent_rope_cache);
  m.def("latent_attention", &latent_attention);
  m.def("latent_attention_mfma", &latent_attention_mfma);
  m.def("causal_conv_silu", &causal_conv_silu);
  m.def("selective_scan", &selective_scan);
  m.def("gdelta_scan", &gdelta_scan);
  m.def("hyper_embed", &hyper_embed);
  m.def("hyper_norm", &hyper_norm);
  m.def("hyper_update_norm", &hyper_update_norm);
  m.def("gated_act", &gated_act);
  m.def("qkv_rope_cache", &qkv_rope_cache);
  m.def("grouped_attention", &grouped_attention);
  m.def("grouped_attention_mfma", &grouped_attention_mfma);
  m.def("moe_route_scores", &moe_route_scores);
  m.def("moe_route", &moe_route);
  m.def("moe_group", &moe_group);
  m.def("moe_gemm", &moe_gemm);
  m.def("moe_combine", &moe_combine);
  m.def("bigram_embed", &bigram_embed);
  m.def("post_norm_add", &post_norm_add);
  m.def("gated_delta_scan", &gated_delta_scan);
  m.def("embed_norm", &embed_norm);
  m.def("rms_norm", &rms_norm);
  m.def("relu2", &relu2);
  m.def("input_conv", &input_conv);
  m.def("hgrn2_scan", &hgrn2_scan);
}
