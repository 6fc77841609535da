// Python bindings of the layer-list decoder kernels (sutro_amd._C_mix).
// Shapes and dtypes are validated here; raw pointers and the current HIP
// stream go to the extern "C" launchers in mix_*.hip. Activation tensors are
// bf16 or fp32 (all of one call the same); recurrence inputs, norm weights
// and the residual stream are fp32.
#include <torch/extension.h>

#include <hip/hip_runtime.h>
#include <c10/hip/HIPStream.h>

#define CHECK_GPU(x) TORCH_CHECK((x).is_cuda(), #x " must be a GPU tensor")
#define CHECK_CONTIG(x) TORCH_CHECK((x).is_contiguous(), #x " must be contiguous")
#define CHECK_F32(x) \
  TORCH_CHECK((x).scalar_type() == at::kFloat, #x " must be fp32")
#define CHECK_I32(x) \
  TORCH_CHECK((x).scalar_type() == at::kInt, #x " must be int32")
#define CHECK_I64(x) \
  TORCH_CHECK((x).scalar_type() == at::kLong, #x " must be int64")

static hipStream_t cur_stream() {
  return c10::hip::getCurrentHIPStream().stream();
}

// 1 = fp32 activations, 0 = bf16
static int act_kind(const torch::Tensor& t) {
  TORCH_CHECK(t.scalar_type() == at::kFloat || t.scalar_type() == at::kBFloat16,
              "activations must be bf16 or fp32");
  return t.scalar_type() == at::kFloat ? 1 : 0;
}

static void check_proj(const torch::Tensor& proj, long off, long width,
                       const char* what) {
  TORCH_CHECK(proj.dim() == 2 && proj.stride(1) == 1, "proj must be [T, N] rows");
  TORCH_CHECK(off >= 0 && off + width <= proj.size(1), what,
              " section outside the projection buffer");
}

extern "C" {
void mix_gelu_tanh_mul(void*, const void*, long, int, int, long, int, int,
                       hipStream_t);
void mix_gated_norm_residual(float*, const void*, const void*, long, int,
                             const float*, float, float, void*, long, int, int,
                             hipStream_t);
void mix_scalar_rmsnorm(void*, const float*, const float*, float, long, int,
                        int, hipStream_t);
void mix_attn_prep(void*, const void*, long, int, int, int, const float*,
                   const float*, float, const float*, int, const long*, void*,
                   void*, const void*, long, const float*, long, int, int, int,
                   int, int, int, hipStream_t);
void mix_local_attention(void*, long, int, const void*, const void*,
                         const void*, const int*, int, const int*, const int*,
                         const int*, float, int, int, const void*, long, int,
                         float, const float*, const float*, int, int, long,
                         long, int, int, int, int, int, int, hipStream_t);
int mix_local_attention_mfma(void*, long, int, const void*, const void*,
                             const void*, const int*, int, const int*,
                             const int*, const int*, const int*, int, float,
                             int, int, const void*, long, int, float,
                             const float*, const float*, int, int, int, int,
                             int, int, int, hipStream_t);
void mix_token_embed(float*, const long*, const long*, const long*,
                     const void*, const void*, long, long, long, const float*,
                     float, long, int, int, hipStream_t);
void mix_dyt_residual(float*, const void*, const float*, const void*,
                      const float*, const void*, const int*, const float*, int,
                      const float*, const float*, const float*, void*, long,
                      int, int, hipStream_t);
void mix_moe_route(int*, float*, const float*, long, int, int, int, int, int,
                   hipStream_t);
void mix_moe_dispatch(int*, int*, int*, int*, const int*, long, int, int, int,
                      long, hipStream_t);
void mix_expert_gemm_plain(void*, const void*, const void*, const int*,
                           const int*, const int*, int, int, int, int, long,
                           int, float, int, hipStream_t);
void sutro_grouped_gemm_glu(void*, const void*, const void*, const int*,
                            const int*, const int*, int, int, int, long, int,
                            float, hipStream_t);
void mix_add_rmsnorm(float*, const void*, const void*, const int*,
                     const float*, int, const float*, const void*, const void*,
                     const void*, long, int, const float*, float, void*, long,
                     int, int, hipStream_t);
void mix_glu_mul(void*, const void*, long, int, int, long, int, int, float,
                 int, hipStream_t);
void mix_moe_route_softmax(int*, float*, float*, const float*, const float*,
                           long, int, int, int, int, int, float, hipStream_t);
void mix_silu_sections(float*, const void*, long, int, int, int, int, int, int,
                       long, int, hipStream_t);
void mix_gated_group_norm(void*, long, int, const float*, const void*, long,
                          int, const float*, float, long, int, int, int, int,
                          hipStream_t);
void mix_ssd_prep(float*, float*, float*, const void*, long, int, int,
                  const float*, const float*, int, const float*, const float*,
                  float*, const int*, const int*, const int*, const int*, long,
                  int, int, int, int, hipStream_t);
int mix_decay_scan(float*, const float*, long, const float*, long,
                   const float*, long, const float*, long, const float*,
                   const float*, float*, const int*, const int*, const int*,
                   int, int, int, int, int, hipStream_t);
void mix_softcap(float*, const void*, float, long, int, hipStream_t);
void sutro_grouped_gemm(void*, const void*, const void*, const int*,
                        const int*, const int*, int, int, int, long, int,
                        int, hipStream_t);
void mix_weighted_rmsnorm(void*, const float*, const float*, float, long, int,
                          int, hipStream_t);
void mix_norm_residual(const float*, const void*, const float*, float, float*,
                       const float*, long, const float*, int, float*,
                       const float*, void*, long, int, int, hipStream_t);
void mix_poly_act(void*, const void*, const float*, float, long, int, int,
                  hipStream_t);
void mix_tied_attn_prep(void*, const void*, long, int, int, const float*,
                        const float*, float, const long*, float, int,
                        const long*, void*, void*, long, int, int, int, int,
                        int, hipStream_t);
void mix_section_rmsnorm(void*, long, const void*, long, int, const float*,
                         float, const long*, long, int, int, hipStream_t);
void mix_sigmoid_gate_mul(void*, long, const void*, long, int, long, int, int,
                          hipStream_t);
void mix_mlstm_scan(float*, float*, float*, float*, const void*, long, int,
                    int, int, int, int, const float*, const float*, float,
                    float*, float*, const int*, const int*, const int*, int,
                    int, int, int, int, hipStream_t);
void mix_mlstm_out(void*, long, int, const float*, const float*, const float*,
                   const void*, long, int, float, long, int, int, int,
                   hipStream_t);
void mix_delta_prep(float*, float*, float*, float*, float*, const void*, long,
                    int, int, int, int, int, const float*, const float*, int,
                    const float*,
                    int, const float*, const float*, float*, const int*,
                    const int*, const int*, const int*, long, int, int, int,
                    int, int, int, hipStream_t);
void mix_delta_scan(float*, const float*, const float*, const float*,
                    const float*, const float*, float*, const int*, const int*,
                    const int*, int, int, int, int, int, hipStream_t);
void mix_delta_out(void*, long, int, const float*, const float*, const void*,
                   long, int, const float*, int, float, float, long, int, int,
                   int, hipStream_t);
}

void gelu_tanh_mul(torch::Tensor out, torch::Tensor proj, long gate_off,
                   long up_off) {
  CHECK_GPU(proj); CHECK_GPU(out); CHECK_CONTIG(out);
  const long T = out.size(0), F = out.size(1);
  TORCH_CHECK(out.scalar_type() == proj.scalar_type(), "dtype mismatch");
  check_proj(proj, gate_off, F, "gate");
  check_proj(proj, up_off, F, "up");
  TORCH_CHECK(proj.size(0) == T, "row mismatch");
  mix_gelu_tanh_mul(out.data_ptr(), proj.data_ptr(), proj.stride(0),
                    (int)gate_off, (int)up_off, T, (int)F, act_kind(proj),
                    cur_stream());
}

void gated_norm_residual(torch::Tensor x, torch::Tensor y, torch::Tensor proj,
                         long gate_off, torch::Tensor gain, double eps,
                         double mult, c10::optional<torch::Tensor> h_out) {
  CHECK_GPU(x); CHECK_CONTIG(x); CHECK_F32(x);
  CHECK_GPU(y); CHECK_CONTIG(y); CHECK_GPU(gain); CHECK_F32(gain);
  const long T = x.size(0), W = x.size(1);
  TORCH_CHECK(y.size(0) == T && y.size(1) == W, "y shape");
  TORCH_CHECK(y.scalar_type() == proj.scalar_type(), "dtype mismatch");
  TORCH_CHECK(proj.size(0) == T, "row mismatch");
  check_proj(proj, gate_off, W, "gate");
  void* hp = nullptr;
  if (h_out.has_value()) {
    CHECK_CONTIG(*h_out);
    TORCH_CHECK(h_out->scalar_type() == y.scalar_type() &&
                h_out->size(0) == T && h_out->size(1) == W, "h_out shape");
    hp = h_out->data_ptr();
  }
  mix_gated_norm_residual(x.data_ptr<float>(), y.data_ptr(), proj.data_ptr(),
                          proj.stride(0), (int)gate_off,
                          gain.data_ptr<float>(), (float)eps, (float)mult, hp,
                          T, (int)W, act_kind(y), cur_stream());
}

void scalar_rmsnorm(torch::Tensor out, torch::Tensor x, torch::Tensor gain,
                    double eps) {
  CHECK_GPU(x); CHECK_CONTIG(x); CHECK_F32(x); CHECK_CONTIG(out);
  CHECK_GPU(gain); CHECK_F32(gain);
  const long W = x.size(-1), T = x.numel() / W;
  TORCH_CHECK(out.numel() == x.numel(), "out shape");
  mix_scalar_rmsnorm(out.data_ptr(), x.data_ptr<float>(),
                     gain.data_ptr<float>(), (float)eps, T, (int)W,
                     act_kind(out), cur_stream());
}

void attn_prep(torch::Tensor q_out, torch::Tensor proj, long q_off, long k_off,
               long v_off, c10::optional<torch::Tensor> q_w,
               c10::optional<torch::Tensor> k_w, double eps,
               torch::Tensor cos_sin, torch::Tensor slots,
               torch::Tensor k_cache,
               torch::Tensor v_cache, c10::optional<torch::Tensor> v_first,
               long v_first_off, c10::optional<torch::Tensor> v_lambda) {
  CHECK_GPU(proj); CHECK_GPU(q_out); CHECK_CONTIG(q_out);
  CHECK_CONTIG(k_cache); CHECK_CONTIG(v_cache);
  CHECK_I64(slots); CHECK_F32(cos_sin); CHECK_CONTIG(cos_sin);
  const long T = q_out.size(0), H = q_out.size(1), dk = q_out.size(2);
  const long G = k_cache.size(1), page = k_cache.size(2);
  const long dv = v_cache.size(3);
  TORCH_CHECK(k_cache.size(3) == dk && v_cache.size(1) == G &&
              v_cache.size(2) == page, "cache shapes");
  TORCH_CHECK(q_out.scalar_type() == proj.scalar_type() &&
              k_cache.scalar_type() == proj.scalar_type() &&
              v_cache.scalar_type() == proj.scalar_type(),
              "q, caches and projections must share one dtype");
  TORCH_CHECK(proj.size(0) == T && slots.numel() == T &&
              cos_sin.dim() == 2 && cos_sin.size(0) == T &&
              cos_sin.size(1) % 2 == 0, "row mismatch");
  check_proj(proj, q_off, H * dk, "q");
  check_proj(proj, k_off, G * dk, "k");
  check_proj(proj, v_off, G * dv, "v");
  const long half = cos_sin.size(1) / 2;
  TORCH_CHECK(2 * half <= dk, "rotated prefix longer than the head");
  TORCH_CHECK(dk <= 256 && dv <= 256, "head sizes above 256 are unsupported");
  const float* qw = nullptr; const float* kw = nullptr;
  if (q_w.has_value()) {
    CHECK_F32(*q_w); TORCH_CHECK(q_w->numel() == dk, "q norm size");
    qw = q_w->data_ptr<float>();
  }
  if (k_w.has_value()) {
    CHECK_F32(*k_w); TORCH_CHECK(k_w->numel() == dk, "k norm size");
    kw = k_w->data_ptr<float>();
  }
  // values blended with another layer's values of the same tokens
  const void* vf = nullptr; long ldvf = 0; const float* vl = nullptr;
  if (v_first.has_value()) {
    TORCH_CHECK(v_lambda.has_value(), "value blending needs its weight");
    CHECK_GPU(*v_first); CHECK_GPU(*v_lambda); CHECK_F32(*v_lambda);
    TORCH_CHECK(v_first->scalar_type() == proj.scalar_type() &&
                v_first->dim() == 2 && v_first->size(0) == T &&
                v_first->stride(1) == 1 && v_lambda->numel() == 1,
                "blended values: dtype or rows");
    check_proj(*v_first, v_first_off, G * dv, "first values");
    vf = (const char*)v_first->data_ptr() +
         v_first_off * (long)v_first->element_size();
    ldvf = v_first->stride(0);
    vl = v_lambda->data_ptr<float>();
  }
  mix_attn_prep(q_out.data_ptr(), proj.data_ptr(), proj.stride(0), (int)q_off,
                (int)k_off, (int)v_off, qw, kw, (float)eps,
                cos_sin.data_ptr<float>(), (int)half, slots.data_ptr<long>(),
                k_cache.data_ptr(), v_cache.data_ptr(), vf, ldvf, vl, T,
                (int)H, (int)G,
                (int)dk, (int)dv, (int)page, act_kind(proj), cur_stream());
}

void local_attention(torch::Tensor out, long out_off, torch::Tensor q,
                     torch::Tensor k_cache, torch::Tensor v_cache,
                     torch::Tensor bt, torch::Tensor seq_lens,
                     torch::Tensor qlocs, torch::Tensor token_seq,
                     double scale, long chunk, long window, torch::Tensor proj,
                     long gate_off, double out_scale,
                     c10::optional<torch::Tensor> tile_seq,
                     c10::optional<torch::Tensor> tile_q0,
                     long prefill_rows, c10::optional<torch::Tensor> bias_r1,
                     c10::optional<torch::Tensor> bias_r2, bool sink,
                     long keep_first) {
  CHECK_GPU(q); CHECK_CONTIG(q); CHECK_CONTIG(k_cache); CHECK_CONTIG(v_cache);
  CHECK_I32(bt); CHECK_I32(seq_lens); CHECK_I32(qlocs); CHECK_I32(token_seq);
  CHECK_CONTIG(bt);
  const long T = q.size(0), H = q.size(1), dk = q.size(2);
  const long G = k_cache.size(1), page = k_cache.size(2);
  const long dv = v_cache.size(3);
  TORCH_CHECK(k_cache.size(3) == dk, "key size mismatch");
  TORCH_CHECK(H % G == 0, "heads must be a multiple of kv heads");
  TORCH_CHECK(dv <= 512 && dk <= 4096, "unsupported head sizes");
  const float* r1 = nullptr; const float* r2 = nullptr;
  if (bias_r1.has_value()) {
    TORCH_CHECK(bias_r2.has_value(), "distance bias needs r1 and r2");
    CHECK_GPU(*bias_r1); CHECK_F32(*bias_r1); CHECK_CONTIG(*bias_r1);
    CHECK_GPU(*bias_r2); CHECK_F32(*bias_r2); CHECK_CONTIG(*bias_r2);
    TORCH_CHECK(bias_r1->numel() == H && bias_r2->numel() == H,
                "distance bias: one r1 and r2 per head");
    r1 = bias_r1->data_ptr<float>(); r2 = bias_r2->data_ptr<float>();
  }
  TORCH_CHECK(out.dim() == 2 && out.stride(1) == 1 && out.size(0) == T &&
              out_off >= 0 && out_off + H * dv <= out.size(1), "out section");
  TORCH_CHECK(out.scalar_type() == q.scalar_type() &&
              k_cache.scalar_type() == q.scalar_type() &&
              v_cache.scalar_type() == q.scalar_type() &&
              proj.scalar_type() == q.scalar_type(), "dtype mismatch");
  TORCH_CHECK(token_seq.numel() == T && qlocs.numel() == seq_lens.numel() + 1 &&
              bt.size(0) == seq_lens.numel(), "batch metadata sizes");
  if (gate_off >= 0) check_proj(proj, gate_off, H, "gate");
  TORCH_CHECK(proj.size(0) == T, "row mismatch");
  // prompt pieces (the first `prefill_rows` rows, tiled 32 rows a tile by
  // tile_seq / tile_q0) go to the MFMA kernel when the shape allows it;
  // single-token rows and every other shape go to the generic kernel
  long t0 = 0;
  if (act_kind(q) == 0 && tile_seq.has_value() && tile_q0.has_value() &&
      prefill_rows > 0) {
    CHECK_I32(*tile_seq); CHECK_I32(*tile_q0);
    TORCH_CHECK(tile_seq->numel() == tile_q0->numel() && prefill_rows <= T,
                "tile map sizes");
    if (mix_local_attention_mfma(
            out.data_ptr(), out.stride(0), (int)out_off, q.data_ptr(),
            k_cache.data_ptr(), v_cache.data_ptr(), bt.data_ptr<int>(),
            (int)bt.size(1), seq_lens.data_ptr<int>(), qlocs.data_ptr<int>(),
            tile_seq->data_ptr<int>(), tile_q0->data_ptr<int>(),
            (int)tile_seq->numel(), (float)scale, (int)chunk, (int)window,
            proj.data_ptr(), proj.stride(0), (int)gate_off, (float)out_scale,
            r1, r2, sink ? 1 : 0, (int)keep_first, (int)H, (int)G, (int)dk,
            (int)dv, (int)page, cur_stream()))
      t0 = prefill_rows;
  }
  if (t0 < T)
    mix_local_attention(out.data_ptr(), out.stride(0), (int)out_off,
                        q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(),
                        bt.data_ptr<int>(), (int)bt.size(1),
                        seq_lens.data_ptr<int>(), qlocs.data_ptr<int>(),
                        token_seq.data_ptr<int>(), (float)scale, (int)chunk,
                        (int)window, proj.data_ptr(), proj.stride(0),
                        (int)gate_off, (float)out_scale, r1, r2, sink ? 1 : 0,
                        (int)keep_first, t0, T - t0, (int)H,
                        (int)G, (int)dk, (int)dv, (int)page, act_kind(q),
                        cur_stream());
}

void delta_prep(torch::Tensor qn, torch::Tensor kn, torch::Tensor v,
                torch::Tensor decay, torch::Tensor beta, torch::Tensor proj,
                long q_off, long k_off, long v_off, long b_off, long a1_off,
                torch::Tensor conv_w, torch::Tensor a2, torch::Tensor dt_bias,
                torch::Tensor a_log, torch::Tensor conv_state,
                torch::Tensor state_slots, torch::Tensor qlocs,
                torch::Tensor seq_lens, torch::Tensor token_seq,
                c10::optional<torch::Tensor> conv_wt) {
  CHECK_GPU(proj);
  const float* wt = nullptr;
  if (conv_wt.has_value()) {  // the filter transposed: [taps, channels]
    CHECK_F32(*conv_wt); CHECK_CONTIG(*conv_wt);
    TORCH_CHECK(conv_wt->dim() == 2 && conv_wt->size(0) == conv_w.size(1) &&
                conv_wt->size(1) == conv_w.size(0), "transposed filter shape");
    wt = conv_wt->data_ptr<float>();
  }
  CHECK_F32(qn); CHECK_F32(kn); CHECK_F32(v); CHECK_F32(decay); CHECK_F32(beta);
  CHECK_CONTIG(qn); CHECK_CONTIG(kn); CHECK_CONTIG(v); CHECK_CONTIG(decay);
  CHECK_CONTIG(beta);
  CHECK_F32(conv_w); CHECK_F32(a2); CHECK_F32(dt_bias); CHECK_F32(a_log);
  CHECK_F32(conv_state); CHECK_CONTIG(conv_w); CHECK_CONTIG(a2);
  CHECK_CONTIG(conv_state);
  CHECK_I32(state_slots); CHECK_I32(qlocs); CHECK_I32(seq_lens);
  CHECK_I32(token_seq);
  const long T = v.size(0), H = v.size(1), dv = v.size(2);
  const long G = qn.size(1), dk = qn.size(2);
  const long S = seq_lens.numel();
  const long C = 2 * G * dk + H * dv, taps = conv_w.size(1);
  const long rank = a2.size(0);  // a2 arrives transposed: [rank, H*dk]
  TORCH_CHECK(dk <= 256 && dv <= 256, "head sizes above 256 are unsupported");
  TORCH_CHECK(H % G == 0, "heads must be a multiple of kv heads");
  TORCH_CHECK(conv_w.size(0) == C, "filter channels");
  TORCH_CHECK(a2.size(1) == H * dk && dt_bias.numel() == H * dk &&
              a_log.numel() == H, "decay parameter sizes");
  TORCH_CHECK(conv_state.dim() == 3 && conv_state.size(2) == C &&
              conv_state.size(1) >= taps - 1 &&
              (taps == 1 || conv_state.size(1) == taps - 1),
              "filter state shape");
  TORCH_CHECK(proj.size(0) == T && token_seq.numel() == T &&
              qlocs.numel() == S + 1 && state_slots.numel() == S &&
              kn.size(0) == T && decay.size(0) == T && beta.size(0) == T,
              "batch metadata sizes");
  check_proj(proj, q_off, G * dk, "q");
  check_proj(proj, k_off, G * dk, "k");
  check_proj(proj, v_off, H * dv, "v");
  check_proj(proj, b_off, H, "beta");
  check_proj(proj, a1_off, rank, "decay input");
  mix_delta_prep(qn.data_ptr<float>(), kn.data_ptr<float>(),
                 v.data_ptr<float>(), decay.data_ptr<float>(),
                 beta.data_ptr<float>(), proj.data_ptr(), proj.stride(0),
                 (int)q_off, (int)k_off, (int)v_off, (int)b_off, (int)a1_off,
                 conv_w.data_ptr<float>(), wt, (int)taps, a2.data_ptr<float>(),
                 (int)rank, dt_bias.data_ptr<float>(), a_log.data_ptr<float>(),
                 conv_state.data_ptr<float>(), state_slots.data_ptr<int>(),
                 qlocs.data_ptr<int>(), seq_lens.data_ptr<int>(),
                 token_seq.data_ptr<int>(), T, (int)S, (int)H, (int)G, (int)dk,
                 (int)dv, act_kind(proj), cur_stream());
}

void delta_scan(torch::Tensor o, torch::Tensor qn, torch::Tensor kn,
                torch::Tensor v, torch::Tensor decay, torch::Tensor beta,
                torch::Tensor ssm, torch::Tensor state_slots,
                torch::Tensor qlocs, torch::Tensor seq_lens) {
  CHECK_GPU(v); CHECK_F32(o); CHECK_F32(qn); CHECK_F32(kn); CHECK_F32(v);
  CHECK_F32(decay); CHECK_F32(beta); CHECK_F32(ssm);
  CHECK_CONTIG(o); CHECK_CONTIG(qn); CHECK_CONTIG(kn); CHECK_CONTIG(v);
  CHECK_CONTIG(decay); CHECK_CONTIG(beta); CHECK_CONTIG(ssm);
  CHECK_I32(state_slots); CHECK_I32(qlocs); CHECK_I32(seq_lens);
  const long T = v.size(0), H = v.size(1), dv = v.size(2);
  const long G = kn.size(1), dk = kn.size(2);
  const long S = seq_lens.numel();
  TORCH_CHECK(dk <= 256, "key size above 256 is unsupported");
  TORCH_CHECK(H % G == 0, "heads must be a multiple of kv heads");
  TORCH_CHECK(ssm.dim() == 4 && ssm.size(1) == H && ssm.size(2) == dk &&
              ssm.size(3) == dv, "state shape");
  TORCH_CHECK(o.numel() == v.numel() && qn.numel() == kn.numel() &&
              kn.size(0) == T && decay.numel() == T * H * dk &&
              beta.numel() == T * H && qlocs.numel() == S + 1 &&
              state_slots.numel() == S, "operand sizes");
  mix_delta_scan(o.data_ptr<float>(), qn.data_ptr<float>(),
                 kn.data_ptr<float>(), v.data_ptr<float>(),
                 decay.data_ptr<float>(), beta.data_ptr<float>(),
                 ssm.data_ptr<float>(), state_slots.data_ptr<int>(),
                 qlocs.data_ptr<int>(), seq_lens.data_ptr<int>(), (int)S,
                 (int)H, (int)G, (int)dk, (int)dv, cur_stream());
}

void delta_out(torch::Tensor out, long out_off, torch::Tensor o,
               torch::Tensor norm_w, torch::Tensor proj, long g1_off,
               torch::Tensor g2, double eps, double out_scale) {
  CHECK_GPU(o); CHECK_F32(o); CHECK_CONTIG(o); CHECK_F32(norm_w);
  CHECK_F32(g2); CHECK_CONTIG(g2);
  const long T = o.size(0), H = o.size(1), dv = o.size(2);
  const long rank = g2.size(0);  // g2 arrives transposed: [rank, H*dv]
  TORCH_CHECK(norm_w.numel() == dv && g2.size(1) == H * dv, "parameter sizes");
  TORCH_CHECK(out.dim() == 2 && out.stride(1) == 1 && out.size(0) == T &&
              out_off >= 0 && out_off + H * dv <= out.size(1), "out section");
  TORCH_CHECK(out.scalar_type() == proj.scalar_type(), "dtype mismatch");
  TORCH_CHECK(proj.size(0) == T, "row mismatch");
  check_proj(proj, g1_off, rank, "gate input");
  mix_delta_out(out.data_ptr(), out.stride(0), (int)out_off,
                o.data_ptr<float>(), norm_w.data_ptr<float>(), proj.data_ptr(),
                proj.stride(0), (int)g1_off, g2.data_ptr<float>(), (int)rank,
                (float)eps, (float)out_scale, T, (int)H, (int)dv,
                act_kind(out), cur_stream());
}

// ---- embedding, sandwich norms with depth-weighted sums, PolyNorm ----

void token_embed(torch::Tensor out, torch::Tensor ids,
                 c10::optional<torch::Tensor> prev, torch::Tensor pos,
                 torch::Tensor embed, c10::optional<torch::Tensor> bigram,
                 long buckets, long mul_prev, long mul_cur,
                 c10::optional<torch::Tensor> inv_freq, double scale) {
  CHECK_GPU(out); CHECK_F32(out); CHECK_CONTIG(out); CHECK_GPU(ids);
  CHECK_I64(ids); CHECK_I64(pos); CHECK_CONTIG(ids); CHECK_CONTIG(pos);
  CHECK_GPU(embed); CHECK_CONTIG(embed);
  const long T = ids.numel(), W = embed.size(1);
  TORCH_CHECK(out.dim() == 2 && out.size(0) == T && out.size(1) == W &&
              pos.numel() == T, "embedding output shape");
  const void* bp = nullptr; const long* pp = nullptr;
  if (bigram.has_value()) {
    TORCH_CHECK(prev.has_value(), "a bigram table needs the previous tokens");
    CHECK_GPU(*bigram); CHECK_CONTIG(*bigram); CHECK_I64(*prev);
    CHECK_CONTIG(*prev);
    TORCH_CHECK(bigram->scalar_type() == embed.scalar_type() &&
                bigram->size(1) == W && bigram->size(0) == buckets + 1 &&
                prev->numel() == T && buckets > 0, "bigram table shape");
    bp = bigram->data_ptr(); pp = prev->data_ptr<long>();
  }
  const float* fp = nullptr;
  if (inv_freq.has_value()) {
    CHECK_GPU(*inv_freq); CHECK_F32(*inv_freq); CHECK_CONTIG(*inv_freq);
    TORCH_CHECK(inv_freq->numel() == (W + 1) / 2, "sinusoid table");
    fp = inv_freq->data_ptr<float>();
  }
  mix_token_embed(out.data_ptr<float>(), ids.data_ptr<long>(), pp,
                  pos.data_ptr<long>(), embed.data_ptr(), bp, buckets,
                  mul_prev, mul_cur, fp, (float)scale, T, (int)W,
                  act_kind(embed), cur_stream());
}

void weighted_rmsnorm(torch::Tensor out, torch::Tensor x, torch::Tensor w,
                      double eps) {
  CHECK_GPU(x); CHECK_CONTIG(x); CHECK_F32(x); CHECK_GPU(out);
  CHECK_CONTIG(out); CHECK_GPU(w); CHECK_F32(w); CHECK_CONTIG(w);
  const long W = x.size(-1), T = x.numel() / W;
  TORCH_CHECK(out.numel() == x.numel() && w.numel() == W, "norm shapes");
  mix_weighted_rmsnorm(out.data_ptr(), x.data_ptr<float>(),
                       w.data_ptr<float>(), (float)eps, T, (int)W,
                       act_kind(out), cur_stream());
}

void norm_residual(torch::Tensor x_in, torch::Tensor y, torch::Tensor w_post,
                   double eps, torch::Tensor x_out,
                   c10::optional<torch::Tensor> stack,
                   c10::optional<torch::Tensor> depth_w,
                   c10::optional<torch::Tensor> mix_out,
                   c10::optional<torch::Tensor> next_w,
                   c10::optional<torch::Tensor> h_out) {
  CHECK_GPU(x_in); CHECK_F32(x_in); CHECK_CONTIG(x_in);
  CHECK_GPU(x_out); CHECK_F32(x_out); CHECK_CONTIG(x_out);
  CHECK_GPU(y); CHECK_CONTIG(y); CHECK_GPU(w_post); CHECK_F32(w_post);
  CHECK_CONTIG(w_post);
  TORCH_CHECK(x_in.dim() == 2, "x_in must be [T, W]");
  const long T = x_in.size(0), W = x_in.size(1);
  TORCH_CHECK(y.dim() == 2 && y.size(0) == T && y.size(1) == W &&
              x_out.numel() == T * W && w_post.numel() == W, "row shapes");
  const float* sp = nullptr; const float* dp = nullptr; float* mp = nullptr;
  long stride = 0; int nd = 0;
  if (depth_w.has_value()) {
    TORCH_CHECK(stack.has_value() && mix_out.has_value(),
                "a depth-weighted sum needs the kept results and an output");
    CHECK_GPU(*stack); CHECK_F32(*stack); CHECK_CONTIG(*stack);
    CHECK_GPU(*depth_w); CHECK_F32(*depth_w); CHECK_CONTIG(*depth_w);
    CHECK_GPU(*mix_out); CHECK_F32(*mix_out); CHECK_CONTIG(*mix_out);
    nd = (int)depth_w->numel();
    TORCH_CHECK(stack->dim() == 3 && stack->size(1) == T &&
                stack->size(2) == W && nd >= 1 && stack->size(0) >= nd &&
                mix_out->numel() == T * W, "kept-results shape");
    // the newest kept result is the row this call writes
    TORCH_CHECK(x_out.data_ptr<float>() ==
                stack->data_ptr<float>() + (long)(nd - 1) * T * W,
                "x_out must be entry len(depth_w)-1 of the kept results");
    sp = stack->data_ptr<float>(); dp = depth_w->data_ptr<float>();
    mp = mix_out->data_ptr<float>(); stride = T * W;
  }
  const float* np_ = nullptr; void* hp = nullptr;
  if (next_w.has_value()) {
    TORCH_CHECK(h_out.has_value(), "next_w needs h_out");
    CHECK_GPU(*next_w); CHECK_F32(*next_w); CHECK_CONTIG(*next_w);
    CHECK_GPU(*h_out); CHECK_CONTIG(*h_out);
    TORCH_CHECK(next_w->numel() == W && h_out->numel() == T * W &&
                h_out->scalar_type() == y.scalar_type(), "h_out shape");
    np_ = next_w->data_ptr<float>(); hp = h_out->data_ptr();
  }
  mix_norm_residual(x_in.data_ptr<float>(), y.data_ptr(),
                    w_post.data_ptr<float>(), (float)eps,
                    x_out.data_ptr<float>(), sp, stride, dp, nd, mp, np_, hp,
                    T, (int)W, act_kind(y), cur_stream());
}

void poly_act(torch::Tensor out, torch::Tensor z, torch::Tensor coef,
              double eps) {
  CHECK_GPU(z); CHECK_CONTIG(z); CHECK_GPU(out); CHECK_CONTIG(out);
  CHECK_GPU(coef); CHECK_F32(coef); CHECK_CONTIG(coef);
  TORCH_CHECK(z.dim() == 2 && out.sizes() == z.sizes() &&
              out.scalar_type() == z.scalar_type() && coef.numel() == 4,
              "activation shapes");
  mix_poly_act(out.data_ptr(), z.data_ptr(), coef.data_ptr<float>(),
               (float)eps, z.size(0), (int)z.size(1), act_kind(z),
               cur_stream());
}

// ---- whole-projection norms: tied-value attention prep, latents, gates ----

void tied_attn_prep(torch::Tensor q_out, torch::Tensor proj, long q_off,
                    long k_off, torch::Tensor q_w, torch::Tensor k_w,
                    double eps, torch::Tensor pos, double temp_coef,
                    long temp_every, torch::Tensor slots,
                    torch::Tensor k_cache, torch::Tensor v_cache) {
  CHECK_GPU(proj); CHECK_GPU(q_out); CHECK_CONTIG(q_out);
  CHECK_GPU(k_cache); CHECK_GPU(v_cache);
  CHECK_CONTIG(k_cache); CHECK_CONTIG(v_cache);
  CHECK_I64(slots); CHECK_I64(pos); CHECK_CONTIG(slots); CHECK_CONTIG(pos);
  CHECK_GPU(q_w); CHECK_F32(q_w); CHECK_CONTIG(q_w);
  CHECK_GPU(k_w); CHECK_F32(k_w); CHECK_CONTIG(k_w);
  const long T = q_out.size(0), H = q_out.size(1), dk = q_out.size(2);
  const long G = k_cache.size(1), page = k_cache.size(2);
  TORCH_CHECK(k_cache.dim() == 4 && k_cache.size(3) == dk &&
              v_cache.sizes() == k_cache.sizes(),
              "values are the keys: both caches must be [blocks, G, page, dk]");
  TORCH_CHECK(q_out.scalar_type() == proj.scalar_type() &&
              k_cache.scalar_type() == proj.scalar_type() &&
              v_cache.scalar_type() == proj.scalar_type(),
              "q, caches and projections must share one dtype");
  TORCH_CHECK(proj.size(0) == T && slots.numel() == T && pos.numel() == T,
              "row mismatch");
  TORCH_CHECK(q_w.numel() == H * dk && k_w.numel() == G * dk, "norm sizes");
  check_proj(proj, q_off, H * dk, "q");
  check_proj(proj, k_off, G * dk, "k");
  mix_tied_attn_prep(q_out.data_ptr(), proj.data_ptr(), proj.stride(0),
                     (int)q_off, (int)k_off, q_w.data_ptr<float>(),
                     k_w.data_ptr<float>(), (float)eps, pos.data_ptr<long>(),
                     (float)temp_coef, (int)temp_every, slots.data_ptr<long>(),
                     k_cache.data_ptr(), v_cache.data_ptr(), T, (int)H, (int)G,
                     (int)dk, (int)page, act_kind(proj), cur_stream());
}

void section_rmsnorm(torch::Tensor out, torch::Tensor proj, long off,
                     torch::Tensor w, double eps,
                     c10::optional<torch::Tensor> rows) {
  CHECK_GPU(proj); CHECK_GPU(out); CHECK_GPU(w); CHECK_F32(w); CHECK_CONTIG(w);
  TORCH_CHECK(out.dim() == 2 && out.stride(1) == 1 &&
              out.scalar_type() == proj.scalar_type(), "out must be [N, n] rows");
  const long T = proj.size(0), n = out.size(1);
  TORCH_CHECK(w.numel() == n, "norm size");
  check_proj(proj, off, n, "normed");
  const long* rp = nullptr;
  if (rows.has_value()) {
    CHECK_GPU(*rows); CHECK_I64(*rows); CHECK_CONTIG(*rows);
    TORCH_CHECK(rows->numel() == T, "one destination row per token");
    rp = rows->data_ptr<long>();
  } else {
    TORCH_CHECK(out.size(0) == T, "row mismatch");
  }
  mix_section_rmsnorm(out.data_ptr(), out.stride(0), proj.data_ptr(),
                      proj.stride(0), (int)off, w.data_ptr<float>(),
                      (float)eps, rp, T, (int)n, act_kind(proj), cur_stream());
}

void sigmoid_gate_mul(torch::Tensor v, torch::Tensor proj, long g_off) {
  CHECK_GPU(v); CHECK_GPU(proj);
  TORCH_CHECK(v.dim() == 2 && v.stride(1) == 1 &&
              v.scalar_type() == proj.scalar_type() &&
              proj.size(0) == v.size(0), "gated rows");
  check_proj(proj, g_off, v.size(1), "gate");
  mix_sigmoid_gate_mul(v.data_ptr(), v.stride(0), proj.data_ptr(),
                       proj.stride(0), (int)g_off, v.size(0), (int)v.size(1),
                       act_kind(v), cur_stream());
}

// ---- mLSTM ----

void mlstm_scan(torch::Tensor o, torch::Tensor em, torch::Tensor proj,
                long q_off, long k_off, long v_off, long i_off, long f_off,
                torch::Tensor i_bias, torch::Tensor f_bias, double cap,
                torch::Tensor mem, torch::Tensor mstate,
                torch::Tensor state_slots, torch::Tensor qlocs,
                torch::Tensor seq_lens) {
  CHECK_GPU(proj); CHECK_GPU(o); CHECK_F32(o); CHECK_CONTIG(o);
  CHECK_GPU(em); CHECK_F32(em); CHECK_CONTIG(em);
  CHECK_GPU(mem); CHECK_F32(mem); CHECK_CONTIG(mem);
  CHECK_GPU(mstate); CHECK_F32(mstate); CHECK_CONTIG(mstate);
  CHECK_GPU(i_bias); CHECK_F32(i_bias); CHECK_GPU(f_bias); CHECK_F32(f_bias);
  CHECK_I32(state_slots); CHECK_I32(qlocs); CHECK_I32(seq_lens);
  TORCH_CHECK(mem.dim() == 4 && o.dim() == 3, "state and read-out ranks");
  const long T = proj.size(0), H = mem.size(1), dk = mem.size(2);
  const long dv = mem.size(3) - 1, S = seq_lens.numel();
  TORCH_CHECK(dk <= 256 && dv >= 1, "key size above 256 is unsupported");
  TORCH_CHECK(o.size(0) == T && o.size(1) == H && o.size(2) == dv + 1 &&
              em.numel() == T * H && mstate.dim() == 2 &&
              mstate.size(0) == mem.size(0) && mstate.size(1) == H &&
              i_bias.numel() == H && f_bias.numel() == H &&
              qlocs.numel() == S + 1 && state_slots.numel() == S,
              "operand sizes");
  check_proj(proj, q_off, H * dk, "q");
  check_proj(proj, k_off, H * dk, "k");
  check_proj(proj, v_off, H * dv, "v");
  check_proj(proj, i_off, H, "input gate");
  check_proj(proj, f_off, H, "forget gate");
  auto scratch = torch::empty({2, T, H}, o.options());
  float* fa = scratch.data_ptr<float>();
  mix_mlstm_scan(o.data_ptr<float>(), em.data_ptr<float>(), fa, fa + T * H,
                 proj.data_ptr(), proj.stride(0), (int)q_off, (int)k_off,
                 (int)v_off, (int)i_off, (int)f_off, i_bias.data_ptr<float>(),
                 f_bias.data_ptr<float>(), (float)cap, mem.data_ptr<float>(),
                 mstate.data_ptr<float>(), state_slots.data_ptr<int>(),
                 qlocs.data_ptr<int>(), seq_lens.data_ptr<int>(), (int)S,
                 (int)H, (int)dk, (int)dv, act_kind(proj), cur_stream());
}

void mlstm_out(torch::Tensor out, long out_off, torch::Tensor o,
               torch::Tensor em, torch::Tensor norm_w, torch::Tensor proj,
               long g_off, double eps) {
  CHECK_GPU(o); CHECK_F32(o); CHECK_CONTIG(o); CHECK_GPU(em); CHECK_F32(em);
  CHECK_CONTIG(em); CHECK_GPU(norm_w); CHECK_F32(norm_w); CHECK_CONTIG(norm_w);
  CHECK_GPU(out); CHECK_GPU(proj);
  const long T = o.size(0), H = o.size(1), dv = o.size(2) - 1;
  TORCH_CHECK(norm_w.numel() == H * dv && em.numel() == T * H,
              "parameter sizes");
  TORCH_CHECK(out.dim() == 2 && out.stride(1) == 1 && out.size(0) == T &&
              out_off >= 0 && out_off + H * dv <= out.size(1), "out section");
  TORCH_CHECK(out.scalar_type() == proj.scalar_type() && proj.size(0) == T,
              "dtype or row mismatch");
  check_proj(proj, g_off, H * dv, "gate");
  mix_mlstm_out(out.data_ptr(), out.stride(0), (int)out_off,
                o.data_ptr<float>(), em.data_ptr<float>(),
                norm_w.data_ptr<float>(), proj.data_ptr(), proj.stride(0),
                (int)g_off, (float)eps, T, (int)H, (int)dv, act_kind(out),
                cur_stream());
}

// ---- Dynamic-Tanh residual, routed experts, soft cap ----

static const float* opt_f32(const c10::optional<torch::Tensor>& t, long n,
                            const char* what) {
  if (!t.has_value()) return nullptr;
  TORCH_CHECK(t->is_cuda() && t->scalar_type() == at::kFloat &&
              t->is_contiguous() && t->numel() == n, what,
              ": fp32 GPU tensor of ", n, " values expected");
  return t->data_ptr<float>();
}

void dyt_residual(torch::Tensor x, c10::optional<torch::Tensor> y1,
                  c10::optional<torch::Tensor> ls1,
                  c10::optional<torch::Tensor> y2,
                  c10::optional<torch::Tensor> ls2,
                  c10::optional<torch::Tensor> rows,
                  c10::optional<torch::Tensor> padpos,
                  c10::optional<torch::Tensor> wts,
                  c10::optional<torch::Tensor> alpha,
                  c10::optional<torch::Tensor> nw,
                  c10::optional<torch::Tensor> nb,
                  c10::optional<torch::Tensor> h_out) {
  CHECK_GPU(x); CHECK_F32(x); CHECK_CONTIG(x);
  TORCH_CHECK(x.dim() == 2, "x must be [T, W]");
  const long T = x.size(0), W = x.size(1);
  int kind = -1;
  auto act = [&](const c10::optional<torch::Tensor>& t, long r, long c,
                 const char* what) -> const void* {
    if (!t.has_value()) return nullptr;
    TORCH_CHECK(t->is_cuda() && t->is_contiguous() && t->dim() == 2 &&
                (r < 0 || t->size(0) == r) && t->size(1) == c, what,
                ": shape");
    const int k = act_kind(*t);
    TORCH_CHECK(kind < 0 || kind == k, "activation dtypes differ");
    kind = k;
    return t->data_ptr();
  };
  const void* y1p = act(y1, T, W, "y1");
  const void* y2p = act(y2, T, W, "y2");
  const void* rp = act(rows, -1, W, "rows");
  const float* l1 = opt_f32(ls1, W, "ls1");
  const float* l2 = opt_f32(ls2, W, "ls2");
  TORCH_CHECK(!y1p || l1, "y1 needs ls1");
  TORCH_CHECK(!(y2p || rp) || (y1p && l2), "a second branch needs y1 and ls2");
  TORCH_CHECK(!(y2p && rp), "one second branch at most");
  const int* pp = nullptr; const float* wp = nullptr; long k = 0;
  if (rp) {
    TORCH_CHECK(padpos.has_value() && wts.has_value(), "rows need padpos, wts");
    CHECK_GPU(*padpos); CHECK_I32(*padpos); CHECK_CONTIG(*padpos);
    CHECK_GPU(*wts); CHECK_F32(*wts); CHECK_CONTIG(*wts);
    TORCH_CHECK(padpos->dim() == 2 && padpos->size(0) == T &&
                wts->sizes() == padpos->sizes(), "padpos / wts must be [T, k]");
    k = padpos->size(1);
    pp = padpos->data_ptr<int>(); wp = wts->data_ptr<float>();
  }
  void* hp = nullptr;
  const float* ap = nullptr; const float* nwp = nullptr; const float* nbp = nullptr;
  if (h_out.has_value()) {
    CHECK_GPU(*h_out); CHECK_CONTIG(*h_out);
    TORCH_CHECK(h_out->dim() == 2 && h_out->size(0) == T && h_out->size(1) == W,
                "h_out shape");
    const int hk = act_kind(*h_out);
    TORCH_CHECK(kind < 0 || kind == hk, "activation dtypes differ");
    kind = hk;
    hp = h_out->data_ptr();
    ap = opt_f32(alpha, 1, "alpha");
    nwp = opt_f32(nw, W, "norm weight");
    nbp = opt_f32(nb, W, "norm bias");
    TORCH_CHECK(ap && nwp && nbp, "h_out needs alpha, weight and bias");
  }
  if (kind < 0) return;   // nothing to do
  mix_dyt_residual(x.data_ptr<float>(), y1p, l1, y2p, l2, rp, pp, wp, (int)k,
                   ap, nwp, nbp, hp, T, (int)W, kind, cur_stream());
}

void moe_route(torch::Tensor idx, torch::Tensor wts, torch::Tensor logits,
               long groups, long keep, long rank) {
  CHECK_GPU(logits); CHECK_F32(logits); CHECK_CONTIG(logits);
  CHECK_GPU(idx); CHECK_I32(idx); CHECK_CONTIG(idx);
  CHECK_GPU(wts); CHECK_F32(wts); CHECK_CONTIG(wts);
  TORCH_CHECK(logits.dim() == 2 && idx.dim() == 2, "router shapes");
  const long T = logits.size(0), E = logits.size(1), top = idx.size(1);
  TORCH_CHECK(idx.size(0) == T && wts.sizes() == idx.sizes(), "router shapes");
  TORCH_CHECK(groups >= 1 && groups <= 1024 && E % groups == 0 && keep >= 1 &&
              keep <= groups && rank >= 1, "router groups");
  TORCH_CHECK(top >= 1 && top <= keep * (E / groups),
              "more choices than the kept groups hold");
  TORCH_CHECK(4 * (E + groups) * 4 <= 64 * 1024, "too many experts");
  mix_moe_route(idx.data_ptr<int>(), wts.data_ptr<float>(),
                logits.data_ptr<float>(), T, (int)E, (int)top, (int)groups,
                (int)keep, (int)rank, cur_stream());
}

void moe_dispatch(torch::Tensor row_tok, torch::Tensor tile_off,
                  torch::Tensor counts, torch::Tensor padpos,
                  torch::Tensor idx, long bm) {
  CHECK_GPU(idx); CHECK_I32(idx); CHECK_CONTIG(idx);
  CHECK_GPU(row_tok); CHECK_I32(row_tok); CHECK_CONTIG(row_tok);
  CHECK_GPU(tile_off); CHECK_I32(tile_off); CHECK_CONTIG(tile_off);
  CHECK_GPU(counts); CHECK_I32(counts); CHECK_CONTIG(counts);
  CHECK_GPU(padpos); CHECK_I32(padpos); CHECK_CONTIG(padpos);
  TORCH_CHECK(idx.dim() == 2 && padpos.sizes() == idx.sizes(), "pair shapes");
  const long T = idx.size(0), k = idx.size(1), E = counts.numel();
  TORCH_CHECK(bm == 64 || bm == 128, "bm must be 64 or 128");
  TORCH_CHECK(tile_off.numel() == E + 1 && row_tok.numel() % bm == 0 &&
              row_tok.numel() >= T * k + E * (bm - 1), "segment table sizes");
  TORCH_CHECK((2 * E + 1) * 4 <= 64 * 1024, "too many experts");
  mix_moe_dispatch(row_tok.data_ptr<int>(), tile_off.data_ptr<int>(),
                   counts.data_ptr<int>(), padpos.data_ptr<int>(),
                   idx.data_ptr<int>(), T * k, (int)k, (int)E, (int)bm,
                   row_tok.numel(), cur_stream());
}

void expert_gemm(torch::Tensor out, torch::Tensor a, torch::Tensor w,
                 c10::optional<torch::Tensor> row_tok, torch::Tensor tile_off,
                 torch::Tensor counts, long act, long bm, double limit) {
  CHECK_GPU(a); CHECK_CONTIG(a); CHECK_GPU(w); CHECK_CONTIG(w);
  CHECK_GPU(out); CHECK_CONTIG(out);
  CHECK_I32(tile_off); CHECK_I32(counts); CHECK_GPU(tile_off); CHECK_GPU(counts);
  CHECK_CONTIG(tile_off); CHECK_CONTIG(counts);
  TORCH_CHECK(w.dim() == 3 && a.dim() == 2 && out.dim() == 2, "operand ranks");
  const bool glu = act == 3;   // w rows: gate rows, then up rows
  const long E = w.size(0), K = w.size(2);
  const long N = glu ? w.size(1) / 2 : w.size(1);
  const long n_rows = out.size(0);
  TORCH_CHECK(bm == 64 || bm == 128, "bm must be 64 or 128");
  TORCH_CHECK(act == 0 || act == 2 || act == 3,
              "activation: 0 (none), 2 (relu squared) or 3 (clamped unit)");
  TORCH_CHECK(!glu || (w.size(1) % 2 == 0 && limit > 0),
              "the clamped unit needs gate and up rows and a limit");
  TORCH_CHECK(a.size(1) == K && out.size(1) == N && n_rows % bm == 0 &&
              counts.numel() == E && tile_off.numel() == E + 1,
              "operand shapes");
  const int kind = act_kind(a);
  TORCH_CHECK(act_kind(w) == kind && act_kind(out) == kind, "dtype mismatch");
  const int* rt = nullptr;
  if (row_tok.has_value()) {
    CHECK_GPU(*row_tok); CHECK_I32(*row_tok); CHECK_CONTIG(*row_tok);
    TORCH_CHECK(row_tok->numel() == n_rows, "row table size");
    rt = row_tok->data_ptr<int>();
  } else {
    TORCH_CHECK(a.size(0) == n_rows, "a must be laid out in segments");
  }
  TORCH_CHECK((act != 0) == (rt != nullptr),
              "the gathered stage carries the activation");
  if (kind == 0 && K % 64 == 0 && N % 64 == 0) {
    if (glu)
      sutro_grouped_gemm_glu(out.data_ptr(), a.data_ptr(), w.data_ptr(), rt,
                             tile_off.data_ptr<int>(), counts.data_ptr<int>(),
                             (int)E, (int)(n_rows / bm), (int)N, K, (int)bm,
                             (float)limit, cur_stream());
    else
      sutro_grouped_gemm(out.data_ptr(), a.data_ptr(), w.data_ptr(), rt,
                         tile_off.data_ptr<int>(), counts.data_ptr<int>(),
                         (int)E, (int)(n_rows / bm), (int)N, K, (int)act,
                         (int)bm, cur_stream());
    return;
  }
  mix_expert_gemm_plain(out.data_ptr(), a.data_ptr(), w.data_ptr(), rt,
                        tile_off.data_ptr<int>(), counts.data_ptr<int>(),
                        (int)E, (int)N, (int)K, (int)bm, n_rows,
                        act == 2 ? 1 : (glu ? 2 : 0), (float)limit, kind,
                        cur_stream());
}

// ---- pre-norm layers, decay recurrences ----

static const void* opt_ptr(const c10::optional<torch::Tensor>& t) {
  return t.has_value() ? t->data_ptr() : nullptr;
}

void add_rmsnorm(torch::Tensor x, c10::optional<torch::Tensor> y,
                 c10::optional<torch::Tensor> rows,
                 c10::optional<torch::Tensor> padpos,
                 c10::optional<torch::Tensor> wts,
                 c10::optional<torch::Tensor> idw,
                 c10::optional<torch::Tensor> h_in,
                 c10::optional<torch::Tensor> y2,
                 c10::optional<torch::Tensor> proj2, long sg_off,
                 c10::optional<torch::Tensor> norm_w, double eps,
                 c10::optional<torch::Tensor> h_out) {
  CHECK_GPU(x); CHECK_CONTIG(x); CHECK_F32(x);
  TORCH_CHECK(x.dim() == 2, "x must be [T, W]");
  const long T = x.size(0), W = x.size(1);
  int kind = -1;
  auto act = [&](const torch::Tensor& t, const char* what) {
    CHECK_GPU(t); CHECK_CONTIG(t);
    const int k = act_kind(t);
    TORCH_CHECK(kind < 0 || kind == k, what, ": activation dtypes differ");
    kind = k;
  };
  auto rowsok = [&](const torch::Tensor& t, const char* what) {
    act(t, what);
    TORCH_CHECK(t.dim() == 2 && t.size(0) == T && t.size(1) == W, what,
                " must be [T, W]");
  };
  if (y.has_value()) rowsok(*y, "y");
  if (y2.has_value()) rowsok(*y2, "y2");
  if (h_in.has_value()) rowsok(*h_in, "h_in");
  if (h_out.has_value()) {
    rowsok(*h_out, "h_out");
    TORCH_CHECK(norm_w.has_value(), "a normed output needs the norm weight");
    CHECK_GPU(*norm_w); CHECK_F32(*norm_w); CHECK_CONTIG(*norm_w);
    TORCH_CHECK(norm_w->numel() == W, "norm weight size");
  }
  int k = 0;
  if (rows.has_value()) {
    act(*rows, "rows");
    TORCH_CHECK(padpos.has_value() && wts.has_value(),
                "expert rows need padpos and weights");
    CHECK_GPU(*padpos); CHECK_I32(*padpos); CHECK_CONTIG(*padpos);
    CHECK_GPU(*wts); CHECK_F32(*wts); CHECK_CONTIG(*wts);
    TORCH_CHECK(rows->dim() == 2 && rows->size(1) == W && padpos->dim() == 2 &&
                padpos->size(0) == T && wts->sizes() == padpos->sizes(),
                "expert rows / padpos / weights shapes");
    k = (int)padpos->size(1);
  }
  if (idw.has_value()) {
    CHECK_GPU(*idw); CHECK_F32(*idw); CHECK_CONTIG(*idw);
    TORCH_CHECK(idw->numel() == T && h_in.has_value(),
                "identity weights need one number a token and the input");
  }
  long ld2 = 0;
  if (y2.has_value() && sg_off >= 0) {
    TORCH_CHECK(proj2.has_value(), "the gate of y2 needs its projection");
    CHECK_GPU(*proj2);
    TORCH_CHECK(act_kind(*proj2) == kind && proj2->size(0) == T,
                "gate projection dtype or rows");
    check_proj(*proj2, sg_off, 1, "shared gate");
    ld2 = proj2->stride(0);
  }
  if (kind < 0) kind = 1;
  mix_add_rmsnorm(x.data_ptr<float>(), opt_ptr(y), opt_ptr(rows),
                  (const int*)opt_ptr(padpos), (const float*)opt_ptr(wts), k,
                  idw.has_value() ? (const float*)opt_ptr(idw) : nullptr,
                  idw.has_value() ? opt_ptr(h_in) : nullptr, opt_ptr(y2),
                  (y2.has_value() && sg_off >= 0) ? opt_ptr(proj2) : nullptr,
                  ld2, (int)sg_off, (const float*)opt_ptr(norm_w), (float)eps,
                  h_out.has_value() ? h_out->data_ptr() : nullptr, T, (int)W,
                  kind, cur_stream());
}

void glu_mul(torch::Tensor out, torch::Tensor proj, long gate_off, long up_off,
             long act, double limit) {
  CHECK_GPU(proj); CHECK_GPU(out); CHECK_CONTIG(out);
  const long T = out.size(0), F = out.size(1);
  TORCH_CHECK(out.scalar_type() == proj.scalar_type(), "dtype mismatch");
  TORCH_CHECK(act >= 0 && act <= 2 && (act != 2 || limit > 0),
              "unit: 0 tanh-GELU, 1 silu, 2 clamped (with a limit)");
  check_proj(proj, gate_off, F, "gate");
  check_proj(proj, up_off, F, "up");
  TORCH_CHECK(proj.size(0) == T, "row mismatch");
  mix_glu_mul(out.data_ptr(), proj.data_ptr(), proj.stride(0), (int)gate_off,
              (int)up_off, T, (int)F, (int)act, (float)limit, act_kind(proj),
              cur_stream());
}

void moe_route_softmax(torch::Tensor idx, torch::Tensor wts, torch::Tensor idw,
                       torch::Tensor logits, c10::optional<torch::Tensor> corr,
                       long groups, long keep, long n_real, double scale) {
  CHECK_GPU(logits); CHECK_F32(logits); CHECK_CONTIG(logits);
  CHECK_GPU(idx); CHECK_I32(idx); CHECK_CONTIG(idx);
  CHECK_GPU(wts); CHECK_F32(wts); CHECK_CONTIG(wts);
  CHECK_GPU(idw); CHECK_F32(idw); CHECK_CONTIG(idw);
  TORCH_CHECK(logits.dim() == 2 && idx.dim() == 2, "operand ranks");
  const long T = logits.size(0), n = logits.size(1), top = idx.size(1);
  TORCH_CHECK(idx.size(0) == T && wts.sizes() == idx.sizes() &&
              idw.numel() == T, "output shapes");
  TORCH_CHECK(groups >= 1 && groups <= 1024 && n % groups == 0 && keep >= 1 &&
              keep <= groups && top >= 1 && top <= keep * (n / groups) &&
              n_real >= 0 && n_real <= n && n <= 4096,
              "router shape: groups, kept groups or choices");
  const float* cp = nullptr;
  if (corr.has_value()) {
    CHECK_GPU(*corr); CHECK_F32(*corr); CHECK_CONTIG(*corr);
    TORCH_CHECK(corr->numel() == n, "one correction per router output");
    cp = corr->data_ptr<float>();
  }
  mix_moe_route_softmax(idx.data_ptr<int>(), wts.data_ptr<float>(),
                        idw.data_ptr<float>(), logits.data_ptr<float>(), cp, T,
                        (int)n, (int)n_real, (int)top, (int)groups, (int)keep,
                        (float)scale, cur_stream());
}

void silu_sections(torch::Tensor out, torch::Tensor proj,
                   std::vector<long> offs, std::vector<long> sizes) {
  CHECK_GPU(proj); CHECK_GPU(out); CHECK_F32(out); CHECK_CONTIG(out);
  TORCH_CHECK(offs.size() == sizes.size() && offs.size() >= 1 &&
              offs.size() <= 3, "one to three sections");
  long o[3] = {0, 0, 0}, n[3] = {0, 0, 0}, tot = 0;
  for (size_t i = 0; i < offs.size(); ++i) {
    check_proj(proj, offs[i], sizes[i], "section");
    o[i] = offs[i]; n[i] = sizes[i]; tot += sizes[i];
  }
  const long T = proj.size(0);
  TORCH_CHECK(out.dim() == 2 && out.size(0) == T && out.size(1) == tot,
              "output shape");
  mix_silu_sections(out.data_ptr<float>(), proj.data_ptr(), proj.stride(0),
                    (int)o[0], (int)n[0], (int)o[1], (int)n[1], (int)o[2],
                    (int)n[2], T, act_kind(proj), cur_stream());
}

void gated_group_norm(torch::Tensor out, long out_off, torch::Tensor o,
                      torch::Tensor proj, long g_off, torch::Tensor norm_w,
                      double eps, long groups, bool gate_first) {
  CHECK_GPU(o); CHECK_F32(o); CHECK_CONTIG(o); CHECK_GPU(proj); CHECK_GPU(out);
  CHECK_GPU(norm_w); CHECK_F32(norm_w); CHECK_CONTIG(norm_w);
  const long T = o.size(0);
  const long n = T ? o.numel() / T : norm_w.numel();
  TORCH_CHECK(norm_w.numel() == n && groups >= 1 && n % groups == 0,
              "norm weight size or parts");
  TORCH_CHECK(out.dim() == 2 && out.stride(1) == 1 && out.size(0) == T &&
              out_off >= 0 && out_off + n <= out.size(1), "out section");
  TORCH_CHECK(out.scalar_type() == proj.scalar_type() && proj.size(0) == T,
              "dtype or rows");
  check_proj(proj, g_off, n, "gate");
  mix_gated_group_norm(out.data_ptr(), out.stride(0), (int)out_off,
                       o.data_ptr<float>(), proj.data_ptr(), proj.stride(0),
                       (int)g_off, norm_w.data_ptr<float>(), (float)eps, T,
                       (int)n, (int)groups, gate_first ? 1 : 0, act_kind(proj),
                       cur_stream());
}

void ssd_prep(torch::Tensor xbc, torch::Tensor decay, torch::Tensor dt,
              torch::Tensor proj, long xbc_off, long dt_off,
              torch::Tensor conv_wt, torch::Tensor conv_b,
              torch::Tensor dt_bias, torch::Tensor a_log,
              torch::Tensor conv_state, torch::Tensor state_slots,
              torch::Tensor qlocs, torch::Tensor seq_lens,
              torch::Tensor token_seq) {
  CHECK_GPU(proj); CHECK_GPU(xbc); CHECK_F32(xbc); CHECK_CONTIG(xbc);
  CHECK_F32(decay); CHECK_CONTIG(decay); CHECK_F32(dt); CHECK_CONTIG(dt);
  CHECK_GPU(conv_wt); CHECK_F32(conv_wt); CHECK_CONTIG(conv_wt);
  CHECK_GPU(conv_b); CHECK_F32(conv_b); CHECK_CONTIG(conv_b);
  CHECK_GPU(dt_bias); CHECK_F32(dt_bias); CHECK_GPU(a_log); CHECK_F32(a_log);
  CHECK_GPU(conv_state); CHECK_F32(conv_state); CHECK_CONTIG(conv_state);
  CHECK_I32(state_slots); CHECK_I32(qlocs); CHECK_I32(seq_lens);
  CHECK_I32(token_seq);
  const long T = proj.size(0), C = xbc.size(1), H = decay.size(1);
  const long taps = conv_wt.size(0), S = seq_lens.numel();
  TORCH_CHECK(xbc.size(0) == T && decay.size(0) == T && dt.sizes() ==
              decay.sizes() && conv_wt.dim() == 2 && conv_wt.size(1) == C &&
              conv_b.numel() == C && dt_bias.numel() == H &&
              a_log.numel() == H, "operand shapes");
  TORCH_CHECK(conv_state.dim() == 3 && conv_state.size(2) == C &&
              conv_state.size(1) == std::max<long>(1, taps - 1),
              "filter history shape");
  TORCH_CHECK(token_seq.numel() == T && qlocs.numel() == S + 1 &&
              state_slots.numel() == S, "batch metadata sizes");
  check_proj(proj, xbc_off, C, "x|B|C");
  check_proj(proj, dt_off, H, "dt");
  mix_ssd_prep(xbc.data_ptr<float>(), decay.data_ptr<float>(),
               dt.data_ptr<float>(), proj.data_ptr(), proj.stride(0),
               (int)xbc_off, (int)dt_off, conv_wt.data_ptr<float>(),
               conv_b.data_ptr<float>(), (int)taps, dt_bias.data_ptr<float>(),
               a_log.data_ptr<float>(), conv_state.data_ptr<float>(),
               state_slots.data_ptr<int>(), qlocs.data_ptr<int>(),
               seq_lens.data_ptr<int>(), token_seq.data_ptr<int>(), T, (int)S,
               (int)C, (int)H, act_kind(proj), cur_stream());
}

void decay_scan(torch::Tensor o, torch::Tensor q, torch::Tensor k,
                torch::Tensor v, torch::Tensor decay,
                c10::optional<torch::Tensor> gain,
                c10::optional<torch::Tensor> skip, torch::Tensor state,
                torch::Tensor state_slots, torch::Tensor qlocs,
                torch::Tensor seq_lens) {
  CHECK_GPU(o); CHECK_F32(o); CHECK_CONTIG(o);
  CHECK_GPU(q); CHECK_F32(q); CHECK_GPU(k); CHECK_F32(k);
  CHECK_GPU(v); CHECK_F32(v); CHECK_GPU(decay); CHECK_F32(decay);
  CHECK_CONTIG(decay);
  CHECK_GPU(state); CHECK_F32(state); CHECK_CONTIG(state);
  CHECK_I32(state_slots); CHECK_I32(qlocs); CHECK_I32(seq_lens);
  TORCH_CHECK(q.dim() == 3 && k.dim() == 3 && v.dim() == 3, "q, k, v ranks");
  const long T = v.size(0), H = v.size(1), dv = v.size(2);
  const long G = k.size(1), dk = k.size(2), S = seq_lens.numel();
  // rows may be strided (views of one buffer); heads and channels are dense
  auto dense = [](const torch::Tensor& t) {
    return t.stride(2) == 1 && t.stride(1) == t.size(2);
  };
  TORCH_CHECK(dense(q) && dense(k) && dense(v), "heads must be dense");
  TORCH_CHECK(q.sizes() == k.sizes() && q.size(0) == T && H % G == 0 &&
              o.size(0) == T && o.size(1) == H && o.size(2) == dv,
              "q / k / v / o shapes");
  TORCH_CHECK(state.dim() == 4 && state.size(1) == H && state.size(2) == dk &&
              state.size(3) == dv, "state shape");
  TORCH_CHECK(qlocs.numel() == S + 1 && state_slots.numel() == S,
              "batch metadata sizes");
  long lda = 0;
  if (decay.dim() == 2) {
    TORCH_CHECK(decay.size(0) == T && decay.size(1) == H, "decay shape");
    lda = H;
  } else {
    TORCH_CHECK(decay.dim() == 1 && decay.numel() == H, "decay shape");
  }
  const float* gp = nullptr; const float* sp = nullptr;
  if (gain.has_value()) {
    CHECK_GPU(*gain); CHECK_F32(*gain); CHECK_CONTIG(*gain);
    TORCH_CHECK(gain->numel() == T * H, "gain shape");
    gp = gain->data_ptr<float>();
  }
  if (skip.has_value()) {
    CHECK_GPU(*skip); CHECK_F32(*skip); CHECK_CONTIG(*skip);
    TORCH_CHECK(skip->numel() == H, "skip shape");
    sp = skip->data_ptr<float>();
  }
  if (T == 0) return;
  const int ok = mix_decay_scan(
      o.data_ptr<float>(), q.data_ptr<float>(), q.stride(0),
      k.data_ptr<float>(), k.stride(0), v.data_ptr<float>(), v.stride(0),
      decay.data_ptr<float>(), lda, gp, sp, state.data_ptr<float>(),
      state_slots.data_ptr<int>(), qlocs.data_ptr<int>(),
      seq_lens.data_ptr<int>(), (int)S, (int)H, (int)G, (int)dk, (int)dv,
      cur_stream());
  TORCH_CHECK(ok, "decay_scan: key size above 256 is unsupported");
}

void softcap(torch::Tensor out, torch::Tensor z, double cap) {
  CHECK_GPU(z); CHECK_CONTIG(z); CHECK_GPU(out); CHECK_F32(out);
  CHECK_CONTIG(out);
  TORCH_CHECK(out.numel() == z.numel() && cap > 0, "softcap operands");
  mix_softcap(out.data_ptr<float>(), z.data_ptr(), (float)cap, z.numel(),
              act_kind(z), cur_stream());
}

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.def("add_rmsnorm", &add_rmsnorm,
        "x += y + expert rows + identity share + gated y2; h = rmsnorm(x) * w");
  m.def("glu_mul", &glu_mul, "act(gate) * up: tanh-GELU, silu or clamped unit");
  m.def("moe_route_softmax", &moe_route_softmax,
        "softmax router: correction, group-limited choice, identity experts");
  m.def("silu_sections", &silu_sections, "fp32 silu of projection sections");
  m.def("gated_group_norm", &gated_group_norm,
        "gated read-out normed in equal parts");
  m.def("ssd_prep", &ssd_prep, "Mamba-2 inputs: filter, silu, step, decay");
  m.def("decay_scan", &decay_scan, "S <- a S + b k v^T; o = S^T q + skip v");
  m.def("gelu_tanh_mul", &gelu_tanh_mul, "tanh-GELU(gate) * up");
  m.def("gated_norm_residual", &gated_norm_residual,
        "x += m * g * n(y * sigmoid(gate)); h = cast(x)");
  m.def("scalar_rmsnorm", &scalar_rmsnorm, "RMS norm with one scalar gain");
  m.def("attn_prep", &attn_prep,
        "q/k norm + partial rotation + value blending + paged K/V write",
        py::arg("q"), py::arg("proj"), py::arg("q_off"), py::arg("k_off"),
        py::arg("v_off"), py::arg("q_w"), py::arg("k_w"), py::arg("eps"),
        py::arg("cos_sin"), py::arg("slots"), py::arg("k_cache"),
        py::arg("v_cache"), py::arg("v_first") = c10::nullopt,
        py::arg("v_first_off") = 0, py::arg("v_lambda") = c10::nullopt);
  m.def("local_attention", &local_attention,
        "chunked/windowed paged attention with per-head output gate",
        py::arg("out"), py::arg("out_off"), py::arg("q"), py::arg("k_cache"),
        py::arg("v_cache"), py::arg("bt"), py::arg("seq_lens"),
        py::arg("qlocs"), py::arg("token_seq"), py::arg("scale"),
        py::arg("chunk"), py::arg("window"), py::arg("proj"),
        py::arg("gate_off"), py::arg("out_scale"),
        py::arg("tile_seq") = c10::nullopt, py::arg("tile_q0") = c10::nullopt,
        py::arg("prefill_rows") = 0, py::arg("bias_r1") = c10::nullopt,
        py::arg("bias_r2") = c10::nullopt, py::arg("sink") = false,
        py::arg("keep_first") = 0);
  m.def("delta_prep", &delta_prep, "delta-rule inputs: filters, norms, gates",
        py::arg("qn"), py::arg("kn"), py::arg("v"), py::arg("decay"),
        py::arg("beta"), py::arg("proj"), py::arg("q_off"), py::arg("k_off"),
        py::arg("v_off"), py::arg("b_off"), py::arg("a1_off"),
        py::arg("conv_w"), py::arg("a2"), py::arg("dt_bias"), py::arg("a_log"),
        py::arg("conv_state"), py::arg("state_slots"), py::arg("qlocs"),
        py::arg("seq_lens"), py::arg("token_seq"),
        py::arg("conv_wt") = c10::nullopt);
  m.def("delta_scan", &delta_scan, "gated delta rule over new tokens");
  m.def("delta_out", &delta_out, "per-head norm + low-rank gate of the read-out");
  m.def("token_embed", &token_embed,
        "scaled token row + hashed-bigram row + position sinusoid, fp32",
        py::arg("out"), py::arg("ids"), py::arg("prev"), py::arg("pos"),
        py::arg("embed"), py::arg("bigram"), py::arg("buckets"),
        py::arg("mul_prev"), py::arg("mul_cur"), py::arg("inv_freq"),
        py::arg("scale") = 1.0);
  m.def("weighted_rmsnorm", &weighted_rmsnorm, "RMS norm with a weight vector");
  m.def("norm_residual", &norm_residual,
        "post-norm + residual (+ depth-weighted sum) (+ next pre-norm)");
  m.def("poly_act", &poly_act, "PolyNorm activation");
  m.def("tied_attn_prep", &tied_attn_prep,
        "whole-projection q/k norm, query temperature, K and raw-K page write");
  m.def("section_rmsnorm", &section_rmsnorm,
        "RMS norm of a projection section, optionally scattered by row index");
  m.def("sigmoid_gate_mul", &sigmoid_gate_mul, "v *= sigmoid(gate section)");
  m.def("mlstm_scan", &mlstm_scan, "mLSTM memory over new tokens");
  m.def("mlstm_out", &mlstm_out, "mLSTM read-out normalisation, norm and gate");
  m.def("dyt_residual", &dyt_residual,
        "layer-scaled parallel residual (second branch dense or gathered "
        "expert rows) + Dynamic-Tanh norm of the result");
  m.def("moe_route", &moe_route,
        "sigmoid router with group-limited choice and normalised weights");
  m.def("moe_dispatch", &moe_dispatch,
        "(token, choice) pairs -> padded per-expert segments");
  m.def("expert_gemm", &expert_gemm,
        "GEMM over padded per-expert segments (matrix cores for bf16 with "
        "64-aligned sizes, plain tiles otherwise)",
        py::arg("out"), py::arg("a"), py::arg("w"), py::arg("row_tok"),
        py::arg("tile_off"), py::arg("counts"), py::arg("act"), py::arg("bm"),
        py::arg("limit") = 0.0);
  m.def("softcap", &softcap, "cap * tanh(z / cap), fp32 out");
}
