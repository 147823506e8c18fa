// Python bindings of the hybrid-family kernels (hybrid.hip). Shapes, dtypes, strides and index ranges that the
// kernels assume are checked here, so a malformed call raises instead of launching.
#include <torch/extension.h>
#include <c10/hip/HIPStream.h>
#include <hip/hip_runtime.h>

extern "C" {
hipError_t kafka_hy_ln_shift(int f32, const float* x, int64_t xs, const void* w, const void* b, float eps, void* out,
                             int64_t os, int T, int d, const void* mu, const int* tok_seg, const int* seg,
                             const float* state, float* last, hipStream_t st);
hipError_t kafka_hy_scatter_rows(float* dst, const int* seg, const float* src, int R, int d, hipStream_t st);
hipError_t kafka_hy_add_ln(int f32, float* x, int64_t xs, const void* y, int64_t ys, const void* w, const void* b,
                           float eps, int T, int d, void* out2, int64_t os, const void* w2, const void* b2,
                           hipStream_t st);
hipError_t kafka_hy_gelu_mul(int f32, const void* gu, int64_t gs, void* out, int64_t T, int F, hipStream_t st);
hipError_t kafka_hy_side_gate(int f32, const void* sg, int64_t ss, const int64_t* tokens, const void* emb, int64_t es,
                              int col0, void* out, int64_t T, int dim, hipStream_t st);
hipError_t kafka_hy_side_dwa(int f32, float* x, const void* y, int64_t ys, const void* sw, float eps, float* stack,
                             int layer, const float* dwa, int64_t T, int d, hipStream_t st);
hipError_t kafka_hy_latent_prep(int f32, const void* qgd, int64_t qs, int T, int H, int dim, int rd, int R, int dkv_off,
                                const void* dkv_w, float eps, const int64_t* positions, const float* cos_sin, int dims,
                                void* cache, void* cache_t, int page, const int64_t* slots, void* q_rot,
                                hipStream_t st);
int kafka_hy_latent_mfma_ok(int page, int R, int rd);
hipError_t kafka_hy_latent_attn_mfma(const void* q_lat, int64_t ql_h, int64_t ql_t, const void* q_rot, int64_t qr_t,
                                     int64_t qr_h, const void* cache, const void* cache_t, int R, int rd,
                                     const int* bt, int bt_stride, const int* items, int n_items,
                                     const int64_t* positions, float scale, void* out, int64_t o_h, int64_t o_t, int H,
                                     int nsplit, float* po, float* pml, int T, int window, const float* sink,
                                     hipStream_t st);
hipError_t kafka_hy_sigmoid_mul(int f32, const void* a, int64_t a_h, int64_t a_t, const void* g, int64_t gs, void* out,
                                int64_t T, int H, int vd, hipStream_t st);
int kafka_hy_latent_attn_max_dk();
hipError_t kafka_hy_latent_attn(int f32, const void* q_lat, int64_t ql_h, int64_t ql_t, const void* q_rot, int64_t qr_t,
                                int64_t qr_h, const void* cache, int page, int R, int rd, const int* bt, int bt_stride,
                                const int* tok_seg, const int64_t* positions, float scale, void* out, int64_t o_h,
                                int64_t o_t, int T, int H, int window, const float* sink, hipStream_t st);
hipError_t kafka_hy_short_conv(int f32, const void* proj, int64_t ps, int c0, const void* w, const void* b, int C,
                               int taps, const int* tok_seg, const int* seg, int R, void* state, void* out, int64_t T,
                               int silu, int residual, hipStream_t st);
int kafka_hy_scan_groups(int P, int N);
hipError_t kafka_hy_ssm_scan(int f32, const void* xbc, int64_t xs, const void* proj, int64_t ps, int dt_off,
                             const float* dt_bias, const float* A_log, const float* Dp, int heads, int P, int N, int G,
                             const int* seg, int R, int single, float* state, float* y, int64_t ys, hipStream_t st);
hipError_t kafka_hy_ssm_combine(int f32, const void* proj, int64_t ps, int dt_off, const float* dt_bias,
                                const float* A_log, int heads, int NP_, const int* vseg, const int* cs, int S,
                                float* tmp, float* state, hipStream_t st);
hipError_t kafka_hy_gated_norm(int f32, const float* y, int64_t ys, const void* z, int64_t zs, const void* w, int inner,
                               int groups, float eps, void* out, int64_t os, int64_t T, hipStream_t st);

// gated mixers (hybrid_gated.hip)
hipError_t kafka_hy_rms_norm(int f32, const float* x, int64_t xs, const void* w, float eps, void* out, int64_t os,
                             int T, int d, hipStream_t st);
hipError_t kafka_hy_kv_store(int f32, const void* src, int64_t ss, int k_off, int v_off, int Ck, int Cv, void* kc,
                             void* vt, const int64_t* slots, int64_t T, hipStream_t st);
int kafka_hy_sigmoid_attn_max_d();
int kafka_hy_sigmoid_attn_max_dv();
hipError_t kafka_hy_sigmoid_attn(int f32, const void* q, int64_t qs, int q_off, const void* kc, const void* vt,
                                 const int* bt, int bt_stride, const int* tok_seg, const int64_t* positions, int H,
                                 int G, int D, int Dv, float scale, float softcap, float t_coef, double t_every,
                                 const float* r1, const float* r2, const float* pb, void* out, int64_t os, int64_t T,
                                 hipStream_t st);
int kafka_hy_sigmoid_attn_mfma_ok(int page, int D, int Dv, int rep);
hipError_t kafka_hy_sigmoid_attn_mfma(const void* q, int64_t qs, int q_off, const void* kc, const void* vt,
                                      const int* bt, int bt_stride, const int* items, int n_items,
                                      const int64_t* positions, int H, int G, int D, int Dv, float scale,
                                      float softcap, float t_coef, double t_every, const float* r1, const float* r2,
                                      const float* pb, void* out, int64_t os, int nsplit, float* po, int64_t T,
                                      hipStream_t st);
hipError_t kafka_hy_rglru_scan(int f32, const float* gates, int64_t gs, const void* proj, int64_t ps, const void* u,
                               int64_t us, const float* rate, const int* seg, int R, float* state, void* out,
                               int64_t os, int W, hipStream_t st);
int kafka_hy_rglru_chunk();
hipError_t kafka_hy_rglru_scan_chunked(int f32, float* gates, int64_t gs, const void* proj, int64_t ps, const void* u,
                                       int64_t us, const float* rate, const int* seg, int R, int nch, float* ab,
                                       float* state, void* out, int64_t os, int64_t T, int W, hipStream_t st);
int kafka_hy_mlstm_max_d();
hipError_t kafka_hy_mlstm_scan(int f32, const void* qkv, int64_t qs, const float* gates, int64_t gs, int H, int D,
                               int Dv, float cap, const int* seg, int R, float* S, float* nrm, float* mx, float* out,
                               int64_t os, hipStream_t st);
hipError_t kafka_hy_head_norm_gate(int f32, const float* o, int64_t os_, const void* w, const void* g, int64_t gs,
                                   int g_off, int H, int Dv, float eps, void* out, int64_t outs, int64_t T,
                                   float scale, hipStream_t st);
int kafka_hy_router_max_e();
int kafka_hy_router_max_k();
hipError_t kafka_hy_moe_topk(const float* logits, int64_t ls, int E, int k, float* tw, int* te, int64_t T,
                             hipStream_t st);
int kafka_hy_moe_rows_max_d();
hipError_t kafka_hy_moe_rows(int f32, const void* h, int64_t hs, const void* wgu, const void* wd, const float* tw,
                             const int* te, int d, int F, int k, void* a, float* out, int64_t os, int64_t T,
                             float limit, float alpha, hipStream_t st);
hipError_t kafka_hy_add2(int f32, float* x, int64_t xs, const void* y1, int64_t s1, const void* y2, int64_t s2,
                         int y2_f32, int64_t T, int d, const void* w, float eps, void* out, int64_t os, hipStream_t st);

// residual streams, windowed attention, group-limited router (hybrid_streams.hip)
int kafka_hy_stream_max();
hipError_t kafka_hy_stream_step(float* xs, int64_t s_stride, int64_t t_stride, int S, const void* y, int64_t ys,
                                int y_f32, const void* y2, int64_t y2s, int y2_f32, const float* row_scale,
                                const float* mix, const float* wr, const float* rd, const float* nw, float eps,
                                void* out, int64_t os, int out_f32, float* total, int64_t ts, int64_t T, int d,
                                int center, hipStream_t st);
hipError_t kafka_hy_swish_clamp_mul(int f32, const void* gu, int64_t gs, void* out, int64_t os, int64_t T, int F,
                                    float limit, float alpha, hipStream_t st);
hipError_t kafka_hy_qk_norm_rope_store(int f32, const void* qkv, int64_t qs, int H, int G, int D, int Dv,
                                       const float* qw, const float* kw, float eps, const int64_t* positions,
                                       const float* cos_sin, int dims, const void* vf, int64_t vfs, int vf_off,
                                       float lam, void* kc, void* vt, const int64_t* slots, void* q_out, int64_t qos,
                                       int64_t T, hipStream_t st);
int kafka_hy_window_attn_max_d();
int kafka_hy_window_attn_max_dv();
hipError_t kafka_hy_window_attn(int f32, const void* q, int64_t qs, const void* kc, const void* vt, const int* bt,
                                int bt_stride, const int* tok_seg, const int64_t* positions, int H, int G, int D,
                                int Dv, float scale, int window, const float* sink, void* out, int64_t os, int64_t T,
                                int shared_keys, hipStream_t st);
int kafka_hy_window_attn_mfma_ok(int page, int D, int Dv, int rep);
hipError_t kafka_hy_window_attn_mfma(const void* q, int64_t qs, const void* kc, const void* vt, const int* bt,
                                     int bt_stride, const int* items, int n_items, const int64_t* positions, int H,
                                     int G, int D, int Dv, float scale, int window, const float* sink, void* out,
                                     int64_t os, int nsplit, float* po, float* pml, int64_t T, int shared_keys,
                                     hipStream_t st);
int kafka_hy_grouped_router_max_e();
int kafka_hy_grouped_router_max_k();
int kafka_hy_grouped_router_max_g();
hipError_t kafka_hy_moe_topk_grouped(const float* logits, int64_t ls, int E, int k, const float* corr, int groups,
                                     int keep, float eps, float* tw, int* te, float* gate, int64_t T, hipStream_t st);

// gated recurrences beside attention, rotation + head mix + paged store (hybrid_parallel.hip)
hipError_t kafka_hy_act_norm(int f32, const void* x, int64_t xs, int c0, int n, const float* w, float eps, void* out,
                             int64_t os, int64_t T, int center, hipStream_t st);
hipError_t kafka_hy_gate_mul(int f32, const void* a, int64_t as, const void* g, int64_t gs, int g_off, float scale,
                             void* out, int64_t os, int64_t T, int n, hipStream_t st);
int kafka_hy_mingru_chunk();
hipError_t kafka_hy_mingru_scan(int f32, const void* proj, int64_t ps, const float* bias, const int* seg, int R,
                                float* state, void* out, int64_t os, int W, hipStream_t st);
hipError_t kafka_hy_mingru_scan_chunked(int f32, const void* proj, int64_t ps, const float* bias, const int* seg, int R,
                                        int nch, float* ab, float* ce, float* state, void* out, int64_t os, int64_t T,
                                        int W, hipStream_t st);
int kafka_hy_hgrn2_max_d();
hipError_t kafka_hy_hgrn2_scan(int f32, const void* proj, int64_t ps, int q_off, int f_off, int v_off,
                               const float* f_bias, const float* lower, int H, int D, int Dv, const int* seg, int R,
                               float* S, float* out, int64_t os, hipStream_t st);
hipError_t kafka_hy_hgrn2_decay(int f32, const void* proj, int64_t ps, int f_off, const float* f_bias,
                                const float* lower, int HD, const int* vseg, int n_chunks, float* F, hipStream_t st);
hipError_t kafka_hy_hgrn2_combine(const int* cs, int R, const float* F, int HD, int Dv, float* tmp, float* state,
                                  hipStream_t st);
int kafka_hy_rope_store_max_q();
hipError_t kafka_hy_rope_kv_store(int f32, const void* qkv, int64_t qs, int H, int G, int D, int Dv,
                                  const int64_t* positions, const float* cos_sin, int dims, int pairs,
                                  const float* talk, void* kc, void* vt, const int64_t* slots, void* q_out, int64_t qos,
                                  int64_t T, hipStream_t st);
}

namespace {

#define HY_HIP(e)                                                                     \
  do {                                                                                \
    hipError_t _e = (e);                                                              \
    TORCH_CHECK(_e == hipSuccess, "HIP launch failed: ", hipGetErrorString(_e));      \
  } while (0)

hipStream_t stream() { return c10::hip::getCurrentHIPStream().stream(); }

using OptT = c10::optional<at::Tensor>;

// the activation dtype of a call: every AT tensor must agree
int act_f32(const at::Tensor& t) {
  TORCH_CHECK(t.scalar_type() == at::kFloat || t.scalar_type() == at::kBFloat16, "activations must be bf16 or fp32");
  return t.scalar_type() == at::kFloat;
}
void same_act(int f32, std::initializer_list<const at::Tensor*> ts) {
  for (auto t : ts) TORCH_CHECK(t->is_cuda() && act_f32(*t) == f32, "mixed activation dtypes / not a GPU tensor");
}
void rows2d(const at::Tensor& t, const char* name) {
  TORCH_CHECK(t.is_cuda() && t.dim() == 2 && t.stride(1) == 1, name, ": 2-D GPU tensor with contiguous rows expected");
}
void vec(const at::Tensor& t, int64_t n, const char* name) {
  TORCH_CHECK(t.is_cuda() && t.is_contiguous() && t.numel() == n, name, ": contiguous vector of ", n, " expected");
}
void segs(const at::Tensor& tok_seg, const at::Tensor& seg, int64_t T) {
  TORCH_CHECK(tok_seg.is_cuda() && tok_seg.scalar_type() == at::kInt && tok_seg.is_contiguous() &&
                  tok_seg.numel() == T, "tok_seg: int32 [T]");
  TORCH_CHECK(seg.is_cuda() && seg.scalar_type() == at::kInt && seg.is_contiguous() && seg.dim() == 2 &&
                  seg.size(1) == 4, "seg: int32 [R, 4]");
}

void ln_shift(at::Tensor x, at::Tensor w, at::Tensor b, double eps, at::Tensor out, OptT mu, OptT tok_seg, OptT seg,
              OptT state, OptT last) {
  rows2d(x, "x"); rows2d(out, "out");
  TORCH_CHECK(x.scalar_type() == at::kFloat, "ln_shift: x is the fp32 stream");
  const int f32 = act_f32(out);
  const int64_t T = x.size(0), d = x.size(1);
  same_act(f32, {&w, &b});
  vec(w, d, "w"); vec(b, d, "b");
  TORCH_CHECK(out.size(0) == T && out.size(1) == d, "ln_shift: out shape");
  const void* mup = nullptr; const int *tsp = nullptr, *sgp = nullptr; const float* stp = nullptr; float* lp = nullptr;
  if (mu.has_value()) {
    TORCH_CHECK(tok_seg.has_value() && seg.has_value() && state.has_value() && last.has_value(),
                "ln_shift: a shift needs tok_seg, seg, state and last");
    same_act(f32, {&*mu}); vec(*mu, d, "mu");
    segs(*tok_seg, *seg, T);
    TORCH_CHECK(state->is_cuda() && state->scalar_type() == at::kFloat && state->is_contiguous() && state->dim() == 2 &&
                    state->size(1) == d, "ln_shift: state fp32 [slots, d]");
    TORCH_CHECK(last->is_cuda() && last->scalar_type() == at::kFloat && last->is_contiguous() && last->dim() == 2 &&
                    last->size(0) >= seg->size(0) && last->size(1) == d, "ln_shift: last fp32 [R, d]");
    TORCH_CHECK(x.stride(0) >= d, "ln_shift: rows must not overlap");
    mup = mu->data_ptr(); tsp = tok_seg->data_ptr<int>(); sgp = seg->data_ptr<int>();
    stp = state->data_ptr<float>(); lp = last->data_ptr<float>();
  }
  HY_HIP(kafka_hy_ln_shift(f32, x.data_ptr<float>(), x.stride(0), w.data_ptr(), b.data_ptr(), (float)eps,
                           out.data_ptr(), out.stride(0), (int)T, (int)d, mup, tsp, sgp, stp, lp, stream()));
}

void scatter_rows(at::Tensor dst, at::Tensor seg, at::Tensor src) {
  TORCH_CHECK(dst.is_cuda() && dst.scalar_type() == at::kFloat && dst.is_contiguous() && dst.dim() == 2 &&
                  src.is_cuda() && src.scalar_type() == at::kFloat && src.is_contiguous() && src.dim() == 2 &&
                  src.size(1) == dst.size(1) && seg.is_cuda() && seg.scalar_type() == at::kInt &&
                  seg.is_contiguous() && seg.dim() == 2 && seg.size(1) == 4 && src.size(0) >= seg.size(0),
              "scatter_rows: fp32 [slots, d] <- fp32 [R, d] by int32 seg [R, 4]");
  HY_HIP(kafka_hy_scatter_rows(dst.data_ptr<float>(), seg.data_ptr<int>(), src.data_ptr<float>(), (int)seg.size(0),
                               (int)dst.size(1), stream()));
}

void add_ln(at::Tensor x, at::Tensor y, at::Tensor w, at::Tensor b, double eps, OptT out2, OptT w2, OptT b2) {
  rows2d(x, "x"); rows2d(y, "y");
  TORCH_CHECK(x.scalar_type() == at::kFloat, "add_ln: x is the fp32 stream");
  const int f32 = act_f32(y);
  const int64_t T = x.size(0), d = x.size(1);
  same_act(f32, {&w, &b});
  vec(w, d, "w"); vec(b, d, "b");
  TORCH_CHECK(y.size(0) == T && y.size(1) == d && x.stride(0) >= d, "add_ln: shapes");
  void* o2 = nullptr; int64_t os = 0; const void *w2p = nullptr, *b2p = nullptr;
  if (out2.has_value()) {
    rows2d(*out2, "out2"); same_act(f32, {&*out2});
    TORCH_CHECK(out2->size(0) == T && out2->size(1) == d, "add_ln: out2 shape");
    o2 = out2->data_ptr(); os = out2->stride(0);
    if (w2.has_value()) {
      TORCH_CHECK(b2.has_value(), "add_ln: w2 without b2");
      same_act(f32, {&*w2, &*b2}); vec(*w2, d, "w2"); vec(*b2, d, "b2");
      w2p = w2->data_ptr(); b2p = b2->data_ptr();
    }
  }
  HY_HIP(kafka_hy_add_ln(f32, x.data_ptr<float>(), x.stride(0), y.data_ptr(), y.stride(0), w.data_ptr(), b.data_ptr(),
                         (float)eps, (int)T, (int)d, o2, os, w2p, b2p, stream()));
}

void gelu_mul(at::Tensor gu, at::Tensor out) {
  rows2d(gu, "gu");
  const int f32 = act_f32(gu);
  same_act(f32, {&out});
  TORCH_CHECK(out.is_contiguous() && out.dim() == 2 && out.size(0) == gu.size(0) && gu.size(1) == 2 * out.size(1),
              "gelu_mul: [T, 2F] -> [T, F]");
  HY_HIP(kafka_hy_gelu_mul(f32, gu.data_ptr(), gu.stride(0), out.data_ptr(), gu.size(0), (int)out.size(1), stream()));
}

void side_gate(at::Tensor sg, at::Tensor tokens, at::Tensor emb, int64_t col0, at::Tensor out) {
  rows2d(sg, "sg"); rows2d(emb, "emb");
  const int f32 = act_f32(sg);
  same_act(f32, {&emb, &out});
  const int64_t T = sg.size(0), dim = sg.size(1);
  TORCH_CHECK(tokens.is_cuda() && tokens.scalar_type() == at::kLong && tokens.is_contiguous() && tokens.numel() == T,
              "side_gate: tokens int64 [T]");
  TORCH_CHECK(out.is_contiguous() && out.dim() == 2 && out.size(0) == T && out.size(1) == dim && col0 >= 0 &&
                  col0 + dim <= emb.size(1), "side_gate: shapes");
  HY_HIP(kafka_hy_side_gate(f32, sg.data_ptr(), sg.stride(0), tokens.data_ptr<int64_t>(), emb.data_ptr(),
                            emb.stride(0), (int)col0, out.data_ptr(), T, (int)dim, stream()));
}

void side_dwa(at::Tensor x, OptT y, OptT sw, double eps, OptT stack, int64_t layer, OptT dwa) {
  TORCH_CHECK(x.is_cuda() && x.scalar_type() == at::kFloat && x.is_contiguous() && x.dim() == 2,
              "side_dwa: x fp32 [T, d] contiguous");
  const int64_t T = x.size(0), d = x.size(1);
  int f32 = 0; const void *yp = nullptr, *swp = nullptr; int64_t ys = 0;
  if (y.has_value()) {
    TORCH_CHECK(sw.has_value(), "side_dwa: y without its norm weight");
    rows2d(*y, "y");
    f32 = act_f32(*y);
    same_act(f32, {&*sw}); vec(*sw, d, "side weight");
    TORCH_CHECK(y->size(0) == T && y->size(1) == d, "side_dwa: y shape");
    yp = y->data_ptr(); swp = sw->data_ptr(); ys = y->stride(0);
  }
  float* sp = nullptr; const float* dp = nullptr;
  if (stack.has_value()) {
    TORCH_CHECK(stack->is_cuda() && stack->scalar_type() == at::kFloat && stack->is_contiguous() && stack->dim() == 3 &&
                    stack->size(1) == T && stack->size(2) == d && layer >= 0 && layer + 1 < stack->size(0),
                "side_dwa: stack fp32 [layers + 1, T, d]");
    sp = stack->data_ptr<float>();
    if (dwa.has_value()) {
      TORCH_CHECK(dwa->is_cuda() && dwa->scalar_type() == at::kFloat && dwa->is_contiguous() &&
                      dwa->numel() == layer + 2, "side_dwa: dwa fp32 [layer + 2]");
      dp = dwa->data_ptr<float>();
    }
  }
  HY_HIP(kafka_hy_side_dwa(f32, x.data_ptr<float>(), yp, ys, swp, (float)eps, sp, (int)layer, dp, T, (int)d, stream()));
}

void latent_prep(at::Tensor qgd, int64_t H, int64_t dim, int64_t rd, int64_t R, int64_t dkv_off, OptT dkv_w, double eps,
                 at::Tensor positions, OptT cos_sin, int64_t dims, at::Tensor cache, at::Tensor slots,
                 at::Tensor q_rot, OptT cache_t) {
  rows2d(qgd, "qgd");
  const int f32 = act_f32(qgd);
  same_act(f32, {&cache, &q_rot});
  const int64_t T = qgd.size(0);
  // a model without a rotated part: rd = 0, dims = 0, no table; H = 0: the queries come from elsewhere and only the
  // cache row is written
  TORCH_CHECK(H >= 0 && dim >= 0 && rd >= 0 && dim + rd > 0 && R > 0 && dims >= 0 && dims % 2 == 0 && dims <= rd &&
                  (dims > 0) == (rd > 0) && H * (dim + rd) <= qgd.size(1), "latent_prep: head sizes");
  TORCH_CHECK(cos_sin.has_value() == (dims > 0), "latent_prep: a rotation table comes with rot dims, and only then");
  TORCH_CHECK(positions.is_cuda() && positions.scalar_type() == at::kLong && positions.is_contiguous() &&
                  positions.numel() == T && slots.is_cuda() && slots.scalar_type() == at::kLong &&
                  slots.is_contiguous() && slots.numel() == T, "latent_prep: positions / slots int64 [T]");
  if (dims > 0)
    TORCH_CHECK(cos_sin->is_cuda() && cos_sin->scalar_type() == at::kFloat && cos_sin->is_contiguous() &&
                    cos_sin->dim() == 2 && cos_sin->size(1) == dims, "latent_prep: cos_sin fp32 [positions, dims]");
  TORCH_CHECK(q_rot.is_contiguous() && q_rot.dim() == 3 && q_rot.size(0) == T && q_rot.size(1) == H &&
                  q_rot.size(2) == rd, "latent_prep: q_rot [T, H, rot_dim]");
  TORCH_CHECK(cache.is_contiguous() && cache.dim() == 3 && cache.size(2) == R + rd, "latent_prep: cache [pages, page, "
              "kv_rank + rot_dim]");
  void* ctp = nullptr;
  if (cache_t.has_value()) {
    same_act(f32, {&*cache_t});
    TORCH_CHECK(cache_t->is_contiguous() && cache_t->dim() == 3 && cache_t->size(0) == cache.size(0) &&
                    cache_t->size(1) == R && cache_t->size(2) == cache.size(1),
                "latent_prep: transposed latent copy [pages, kv_rank, page]");
    ctp = cache_t->data_ptr();
  }
  const void* wp = nullptr;
  if (dkv_off >= 0) {
    TORCH_CHECK(dkv_w.has_value() && dkv_off + R + rd <= qgd.size(1), "latent_prep: latent columns");
    same_act(f32, {&*dkv_w}); vec(*dkv_w, R, "latent norm weight");
    wp = dkv_w->data_ptr();
  }
  HY_HIP(kafka_hy_latent_prep(f32, qgd.data_ptr(), qgd.stride(0), (int)T, (int)H, (int)dim, (int)rd, (int)R,
                              (int)dkv_off, wp, (float)eps, positions.data_ptr<int64_t>(),
                              dims > 0 ? cos_sin->data_ptr<float>() : nullptr,
                              (int)dims, cache.data_ptr(), ctp, (int)cache.size(1), slots.data_ptr<int64_t>(),
                              q_rot.data_ptr(), stream()));
}

void sigmoid_mul(at::Tensor a, at::Tensor g, at::Tensor out) {
  const int f32 = act_f32(a);
  same_act(f32, {&g, &out});
  rows2d(g, "g");
  TORCH_CHECK(a.dim() == 3 && a.stride(2) == 1, "sigmoid_mul: a [H, T, v]");
  const int64_t H = a.size(0), T = a.size(1), vd = a.size(2);
  TORCH_CHECK(g.size(0) == T && g.size(1) == H * vd && out.is_contiguous() && out.dim() == 2 && out.size(0) == T &&
                  out.size(1) == H * vd, "sigmoid_mul: shapes");
  HY_HIP(kafka_hy_sigmoid_mul(f32, a.data_ptr(), a.stride(0), a.stride(1), g.data_ptr(), g.stride(0), out.data_ptr(), T,
                              (int)H, (int)vd, stream()));
}

const float* sink_ptr(const OptT& sink, int64_t H) {
  if (!sink.has_value()) return nullptr;
  TORCH_CHECK(sink->is_cuda() && sink->scalar_type() == at::kFloat && sink->is_contiguous() && sink->numel() == H,
              "sink: fp32 [heads]");
  return sink->data_ptr<float>();
}

void latent_attn(at::Tensor q_lat, at::Tensor q_rot, at::Tensor cache, at::Tensor bt, at::Tensor tok_seg,
                 at::Tensor positions, double scale, at::Tensor out, int64_t window, OptT sink) {
  const int f32 = act_f32(q_lat);
  same_act(f32, {&q_rot, &cache, &out});
  TORCH_CHECK(q_lat.dim() == 3 && q_lat.stride(2) == 1 && out.dim() == 3 && out.stride(2) == 1 && q_rot.dim() == 3 &&
                  q_rot.stride(2) == 1, "latent_attn: q_lat / out [H, T, R], q_rot [T, H, rot_dim]");
  const int64_t H = q_lat.size(0), T = q_lat.size(1), R = q_lat.size(2), rd = q_rot.size(2);
  TORCH_CHECK(q_rot.size(0) == T && q_rot.size(1) == H && out.size(0) == H && out.size(1) == T && out.size(2) == R,
              "latent_attn: shapes");
  TORCH_CHECK(cache.is_contiguous() && cache.dim() == 3 && cache.size(2) == R + rd, "latent_attn: cache row");
  TORCH_CHECK(window >= 0, "latent_attn: window");
  TORCH_CHECK(R + rd <= kafka_hy_latent_attn_max_dk(), "latent_attn: kv_rank + rot_dim beyond ",
              kafka_hy_latent_attn_max_dk());
  TORCH_CHECK(bt.is_cuda() && bt.scalar_type() == at::kInt && bt.dim() == 2 && bt.stride(1) == 1 &&
                  tok_seg.is_cuda() && tok_seg.scalar_type() == at::kInt && tok_seg.is_contiguous() &&
                  tok_seg.numel() == T && positions.is_cuda() && positions.scalar_type() == at::kLong &&
                  positions.is_contiguous() && positions.numel() == T, "latent_attn: block tables / tok_seg / positions");
  HY_HIP(kafka_hy_latent_attn(f32, q_lat.data_ptr(), q_lat.stride(0), q_lat.stride(1), q_rot.data_ptr(),
                              q_rot.stride(0), q_rot.stride(1), cache.data_ptr(), (int)cache.size(1), (int)R, (int)rd,
                              bt.data_ptr<int>(), (int)bt.stride(0), tok_seg.data_ptr<int>(),
                              positions.data_ptr<int64_t>(), (float)scale, out.data_ptr(), out.stride(0), out.stride(1),
                              (int)T, (int)H, (int)window, sink_ptr(sink, H), stream()));
}

// the matrix-core kernel: items int32 [n, 4] = (first row, tokens, segment, 0), each at most 32 (token, head) rows of
// one segment (or one token, whose heads go 32 at a time over grid.y)
void latent_attn_mfma(at::Tensor q_lat, at::Tensor q_rot, at::Tensor cache, at::Tensor cache_t, at::Tensor bt,
                      at::Tensor items, int64_t tile_tokens, at::Tensor positions, double scale, at::Tensor out,
                      int64_t nsplit, OptT po, OptT pml, int64_t window, OptT sink) {
  for (const at::Tensor* t : {&q_lat, &q_rot, &cache, &cache_t, &out})
    TORCH_CHECK(t->is_cuda() && t->scalar_type() == at::kBFloat16, "latent_attn_mfma: bf16 GPU tensors");
  TORCH_CHECK(q_lat.dim() == 3 && q_lat.stride(2) == 1 && out.dim() == 3 && out.stride(2) == 1 && q_rot.dim() == 3 &&
                  q_rot.stride(2) == 1, "latent_attn_mfma: q_lat / out [H, T, R], q_rot [T, H, rot_dim]");
  const int64_t H = q_lat.size(0), T = q_lat.size(1), R = q_lat.size(2), rd = q_rot.size(2);
  TORCH_CHECK(q_rot.size(0) == T && q_rot.size(1) == H && out.size(0) == H && out.size(1) == T && out.size(2) == R,
              "latent_attn_mfma: shapes");
  TORCH_CHECK(cache.is_contiguous() && cache.dim() == 3 && cache.size(2) == R + rd && cache_t.is_contiguous() &&
                  cache_t.dim() == 3 && cache_t.size(0) == cache.size(0) && cache_t.size(1) == R &&
                  cache_t.size(2) == cache.size(1), "latent_attn_mfma: cache [pages, 16, R + rd] and [pages, R, 16]");
  TORCH_CHECK(kafka_hy_latent_mfma_ok((int)cache.size(1), (int)R, (int)rd), "latent_attn_mfma: sizes not supported");
  // 16-byte loads: every row start must be a multiple of 8 elements
  TORCH_CHECK(q_lat.stride(0) % 8 == 0 && q_lat.stride(1) % 8 == 0 &&
                  (reinterpret_cast<uintptr_t>(q_lat.data_ptr()) & 15) == 0, "latent_attn_mfma: query alignment");
  TORCH_CHECK(rd == 0 || (q_rot.stride(0) % 8 == 0 && q_rot.stride(1) % 8 == 0 &&
                          (reinterpret_cast<uintptr_t>(q_rot.data_ptr()) & 15) == 0),
              "latent_attn_mfma: rotated query alignment");
  TORCH_CHECK(window >= 0, "latent_attn_mfma: window");
  TORCH_CHECK(tile_tokens >= 1 && tile_tokens * std::min<int64_t>(H, 32) <= 32 && (H <= 32 || tile_tokens == 1),
              "latent_attn_mfma: a tile holds at most 32 (token, head) rows");
  TORCH_CHECK(bt.is_cuda() && bt.scalar_type() == at::kInt && bt.dim() == 2 && bt.stride(1) == 1 && items.is_cuda() &&
                  items.scalar_type() == at::kInt && items.is_contiguous() && items.dim() == 2 && items.size(1) == 4 &&
                  positions.is_cuda() && positions.scalar_type() == at::kLong && positions.is_contiguous() &&
                  positions.numel() == T, "latent_attn_mfma: block tables / items / positions");
  float *pop = nullptr, *pmlp = nullptr;
  TORCH_CHECK(nsplit >= 1 && nsplit <= 64, "latent_attn_mfma: 1..64 key-range splits");
  if (nsplit > 1) {
    TORCH_CHECK(po.has_value() && pml.has_value() && po->is_cuda() && po->scalar_type() == at::kFloat &&
                    po->is_contiguous() && po->numel() >= nsplit * H * T * R && pml->is_cuda() &&
                    pml->scalar_type() == at::kFloat && pml->is_contiguous() && pml->numel() >= nsplit * H * T * 2,
                "latent_attn_mfma: split workspaces fp32 [splits, H, T, R] and [splits, H, T, 2]");
    pop = po->data_ptr<float>(); pmlp = pml->data_ptr<float>();
  }
  HY_HIP(kafka_hy_latent_attn_mfma(q_lat.data_ptr(), q_lat.stride(0), q_lat.stride(1), q_rot.data_ptr(),
                                   q_rot.stride(0), q_rot.stride(1), cache.data_ptr(), cache_t.data_ptr(), (int)R,
                                   (int)rd, bt.data_ptr<int>(), (int)bt.stride(0), items.data_ptr<int>(),
                                   (int)items.size(0), positions.data_ptr<int64_t>(), (float)scale, out.data_ptr(),
                                   out.stride(0), out.stride(1), (int)H, (int)nsplit, pop, pmlp, (int)T, (int)window,
                                   sink_ptr(sink, H), stream()));
}

void short_conv(at::Tensor proj, int64_t c0, at::Tensor w, OptT b, at::Tensor tok_seg, at::Tensor seg,
                at::Tensor state, at::Tensor out, bool silu, bool residual) {
  rows2d(proj, "proj");
  const int f32 = act_f32(proj);
  same_act(f32, {&w, &state, &out});
  const int64_t T = proj.size(0);
  TORCH_CHECK(w.is_contiguous() && w.dim() == 2, "short_conv: w [C, taps]");
  const int64_t C = w.size(0), taps = w.size(1);
  if (b.has_value()) { same_act(f32, {&*b}); vec(*b, C, "conv bias"); }
  segs(tok_seg, seg, T);
  TORCH_CHECK(taps >= 1 && taps <= 16 && c0 >= 0 && c0 + C <= proj.size(1) && out.is_contiguous() && out.dim() == 2 &&
                  out.size(0) == T && out.size(1) == C, "short_conv: shapes");
  TORCH_CHECK(state.is_contiguous() && state.dim() == 3 && state.size(1) == taps - 1 && state.size(2) == C,
              "short_conv: state [slots, taps - 1, C]");
  TORCH_CHECK(out.data_ptr() != proj.data_ptr(), "short_conv: out must not alias the input");
  HY_HIP(kafka_hy_short_conv(f32, proj.data_ptr(), proj.stride(0), (int)c0, w.data_ptr(),
                             b.has_value() ? b->data_ptr() : nullptr, (int)C, (int)taps, tok_seg.data_ptr<int>(),
                             seg.data_ptr<int>(), (int)seg.size(0), state.data_ptr(), out.data_ptr(), T, (int)silu,
                             (int)residual, stream()));
}

void ssm_scan(at::Tensor xbc, at::Tensor proj, int64_t dt_off, at::Tensor dt_bias, at::Tensor A_log, at::Tensor D,
              int64_t heads, int64_t P, int64_t N, int64_t G, at::Tensor seg, at::Tensor state, at::Tensor y) {
  rows2d(xbc, "xbc"); rows2d(proj, "proj"); rows2d(y, "y");
  const int f32 = act_f32(xbc);
  same_act(f32, {&proj});
  const int64_t T = xbc.size(0);
  TORCH_CHECK(heads > 0 && G > 0 && heads % G == 0 && xbc.size(1) == heads * P + 2 * G * N && proj.size(0) == T &&
                  dt_off >= 0 && dt_off + heads <= proj.size(1), "ssm_scan: sizes");
  for (const at::Tensor* t : {&dt_bias, &A_log, &D})
    TORCH_CHECK(t->is_cuda() && t->scalar_type() == at::kFloat && t->is_contiguous() && t->numel() == heads,
                "ssm_scan: dt_bias / A_log / D fp32 [heads]");
  TORCH_CHECK(seg.is_cuda() && seg.scalar_type() == at::kInt && seg.is_contiguous() && seg.dim() == 2 &&
                  seg.size(1) == 4, "ssm_scan: seg int32 [R, 4]");
  TORCH_CHECK(state.is_cuda() && state.scalar_type() == at::kFloat && state.is_contiguous() && state.dim() == 4 &&
                  state.size(1) == heads && state.size(2) == N && state.size(3) == P,
              "ssm_scan: state fp32 [slots, heads, N, P]");
  TORCH_CHECK(y.scalar_type() == at::kFloat && y.size(0) == T && y.size(1) == heads * P, "ssm_scan: y fp32 [T, inner]");
  TORCH_CHECK(kafka_hy_scan_groups((int)P, (int)N) > 0, "ssm_scan: state of ", N, " x ", P, " per head is not supported");
  HY_HIP(kafka_hy_ssm_scan(f32, xbc.data_ptr(), xbc.stride(0), proj.data_ptr(), proj.stride(0), (int)dt_off,
                           dt_bias.data_ptr<float>(), A_log.data_ptr<float>(), D.data_ptr<float>(), (int)heads, (int)P,
                           (int)N, (int)G, seg.data_ptr<int>(), (int)seg.size(0), (int)(T == seg.size(0)),
                           state.data_ptr<float>(),
                           y.data_ptr<float>(), y.stride(0), stream()));
}

// vseg int32 [V, 4] chunk table (first row, rows, -, scratch slot); cs int32 [S, 4] = (first chunk, chunks, first
// position, state slot); at most 256 chunks per segment
void ssm_combine(at::Tensor proj, int64_t dt_off, at::Tensor dt_bias, at::Tensor A_log, int64_t heads, at::Tensor vseg,
                 at::Tensor cs, int64_t max_chunks, at::Tensor tmp, at::Tensor state) {
  rows2d(proj, "proj");
  const int f32 = act_f32(proj);
  TORCH_CHECK(dt_off >= 0 && dt_off + heads <= proj.size(1) && max_chunks >= 1 && max_chunks <= 256,
              "ssm_combine: sizes (at most 256 chunks per segment)");
  for (const at::Tensor* t : {&dt_bias, &A_log})
    TORCH_CHECK(t->is_cuda() && t->scalar_type() == at::kFloat && t->is_contiguous() && t->numel() == heads,
                "ssm_combine: dt_bias / A_log fp32 [heads]");
  for (const at::Tensor* t : {&vseg, &cs})
    TORCH_CHECK(t->is_cuda() && t->scalar_type() == at::kInt && t->is_contiguous() && t->dim() == 2 && t->size(1) == 4,
                "ssm_combine: int32 [n, 4] tables");
  TORCH_CHECK(tmp.is_cuda() && tmp.scalar_type() == at::kFloat && tmp.is_contiguous() && tmp.dim() == 4 &&
                  state.is_cuda() && state.scalar_type() == at::kFloat && state.is_contiguous() && state.dim() == 4 &&
                  tmp.size(0) >= vseg.size(0) && tmp.size(1) == heads && state.size(1) == heads &&
                  tmp.size(2) == state.size(2) && tmp.size(3) == state.size(3), "ssm_combine: state tensors");
  HY_HIP(kafka_hy_ssm_combine(f32, proj.data_ptr(), proj.stride(0), (int)dt_off, dt_bias.data_ptr<float>(),
                              A_log.data_ptr<float>(), (int)heads, (int)(state.size(2) * state.size(3)),
                              vseg.data_ptr<int>(), cs.data_ptr<int>(), (int)cs.size(0), tmp.data_ptr<float>(),
                              state.data_ptr<float>(), stream()));
}

void gated_norm(at::Tensor y, at::Tensor proj, at::Tensor w, int64_t groups, double eps, at::Tensor out) {
  rows2d(y, "y"); rows2d(proj, "proj"); rows2d(out, "out");
  const int f32 = act_f32(proj);
  same_act(f32, {&w, &out});
  const int64_t T = y.size(0), inner = y.size(1);
  TORCH_CHECK(y.scalar_type() == at::kFloat && proj.size(0) == T && proj.size(1) >= inner && groups > 0 &&
                  groups < 65536 && inner % groups == 0 && out.size(0) == T && out.size(1) == inner,
              "gated_norm: shapes");
  vec(w, inner, "norm weight");
  HY_HIP(kafka_hy_gated_norm(f32, y.data_ptr<float>(), y.stride(0), proj.data_ptr(), proj.stride(0), w.data_ptr(),
                             (int)inner, (int)groups, (float)eps, out.data_ptr(), out.stride(0), T, stream()));
}

// ---- gated mixers ----------------------------------------------------------------------------------------------------
void f32t(const at::Tensor& t, const char* name) {
  TORCH_CHECK(t.is_cuda() && t.scalar_type() == at::kFloat, name, ": fp32 GPU tensor expected");
}

void rms_norm(at::Tensor x, at::Tensor w, double eps, at::Tensor out) {
  rows2d(x, "x"); rows2d(out, "out"); f32t(x, "x");
  const int f32 = act_f32(out);
  same_act(f32, {&w});
  const int64_t T = x.size(0), d = x.size(1);
  vec(w, d, "w");
  TORCH_CHECK(out.size(0) == T && out.size(1) == d, "rms_norm: out shape");
  HY_HIP(kafka_hy_rms_norm(f32, x.data_ptr<float>(), x.stride(0), w.data_ptr(), (float)eps, out.data_ptr(),
                           out.stride(0), (int)T, (int)d, stream()));
}

void kv_store(at::Tensor src, int64_t k_off, int64_t v_off, at::Tensor kc, at::Tensor vt, at::Tensor slots) {
  rows2d(src, "src");
  const int f32 = act_f32(src);
  same_act(f32, {&kc, &vt});
  const int64_t T = src.size(0);
  TORCH_CHECK(kc.is_contiguous() && kc.dim() == 3 && kc.size(1) == 16, "kv_store: keys [pages, 16, Ck]");
  TORCH_CHECK(vt.is_contiguous() && vt.dim() == 3 && vt.size(2) == 16 && vt.size(0) == kc.size(0),
              "kv_store: values [pages, Cv, 16]");
  const int64_t Ck = kc.size(2), Cv = vt.size(1);
  TORCH_CHECK(k_off >= 0 && k_off + Ck <= src.size(1) && v_off >= 0 && v_off + Cv <= src.size(1), "kv_store: columns");
  TORCH_CHECK(slots.is_cuda() && slots.scalar_type() == at::kLong && slots.is_contiguous() && slots.numel() == T,
              "kv_store: slots int64 [T]");
  HY_HIP(kafka_hy_kv_store(f32, src.data_ptr(), src.stride(0), (int)k_off, (int)v_off, (int)Ck, (int)Cv, kc.data_ptr(),
                           vt.data_ptr(), slots.data_ptr<int64_t>(), T, stream()));
}

struct SigShape { int64_t T, D, Dv; int f32; };

SigShape sig_check(const at::Tensor& q, int64_t q_off, const at::Tensor& kc, const at::Tensor& vt, const at::Tensor& bt,
                   const at::Tensor& positions, int64_t H, int64_t G, const at::Tensor& r1, const at::Tensor& r2,
                   const at::Tensor& pb, const at::Tensor& out) {
  rows2d(q, "q"); rows2d(out, "out");
  const int f32 = act_f32(q);
  same_act(f32, {&kc, &vt, &out});
  const int64_t T = q.size(0);
  TORCH_CHECK(G >= 1 && H >= 1 && H % G == 0, "sigmoid_attn: heads");
  TORCH_CHECK(kc.is_contiguous() && kc.dim() == 3 && kc.size(1) == 16 && kc.size(2) % G == 0,
              "sigmoid_attn: keys [pages, 16, G D]");
  TORCH_CHECK(vt.is_contiguous() && vt.dim() == 3 && vt.size(2) == 16 && vt.size(0) == kc.size(0) && vt.size(1) % G == 0,
              "sigmoid_attn: values [pages, G Dv, 16]");
  const int64_t D = kc.size(2) / G, Dv = vt.size(1) / G;
  TORCH_CHECK(q_off >= 0 && q_off + H * D <= q.size(1), "sigmoid_attn: query columns");
  TORCH_CHECK(out.size(0) == T && out.size(1) == H * Dv, "sigmoid_attn: out [T, H Dv]");
  TORCH_CHECK(bt.is_cuda() && bt.scalar_type() == at::kInt && bt.dim() == 2 && bt.stride(1) == 1, "sigmoid_attn: bt");
  TORCH_CHECK(positions.is_cuda() && positions.scalar_type() == at::kLong && positions.is_contiguous() &&
                  positions.numel() == T, "sigmoid_attn: positions int64 [T]");
  f32t(r1, "r1"); f32t(r2, "r2"); f32t(pb, "pb");
  vec(r1, H, "r1"); vec(r2, H, "r2"); vec(pb, H, "pb");
  return {T, D, Dv, f32};
}

void sigmoid_attn(at::Tensor q, int64_t q_off, at::Tensor kc, at::Tensor vt, at::Tensor bt, at::Tensor tok_seg,
                  at::Tensor positions, int64_t H, int64_t G, double scale, double softcap, double t_coef,
                  double t_every, at::Tensor r1, at::Tensor r2, at::Tensor pb, at::Tensor out) {
  const SigShape s = sig_check(q, q_off, kc, vt, bt, positions, H, G, r1, r2, pb, out);
  TORCH_CHECK(tok_seg.is_cuda() && tok_seg.scalar_type() == at::kInt && tok_seg.is_contiguous() &&
                  tok_seg.numel() == s.T, "sigmoid_attn: tok_seg int32 [T]");
  TORCH_CHECK(s.D <= kafka_hy_sigmoid_attn_max_d() && s.Dv <= kafka_hy_sigmoid_attn_max_dv(),
              "sigmoid_attn: head sizes up to ", kafka_hy_sigmoid_attn_max_d(), " / ", kafka_hy_sigmoid_attn_max_dv());
  TORCH_CHECK(t_coef == 0.0 || t_every > 0.0, "sigmoid_attn: temperature period");
  HY_HIP(kafka_hy_sigmoid_attn(s.f32, q.data_ptr(), q.stride(0), (int)q_off, kc.data_ptr(), vt.data_ptr(),
                               bt.data_ptr<int>(), (int)bt.stride(0), tok_seg.data_ptr<int>(),
                               positions.data_ptr<int64_t>(), (int)H, (int)G, (int)s.D, (int)s.Dv, (float)scale,
                               (float)softcap, (float)t_coef, t_every, r1.data_ptr<float>(), r2.data_ptr<float>(),
                               pb.data_ptr<float>(), out.data_ptr(), out.stride(0), s.T, stream()));
}

void sigmoid_attn_mfma(at::Tensor q, int64_t q_off, at::Tensor kc, at::Tensor vt, at::Tensor bt, at::Tensor items,
                       int64_t tile_tokens, at::Tensor positions, int64_t H, int64_t G, double scale, double softcap,
                       double t_coef, double t_every, at::Tensor r1, at::Tensor r2, at::Tensor pb, at::Tensor out,
                       int64_t nsplit, OptT po) {
  const SigShape s = sig_check(q, q_off, kc, vt, bt, positions, H, G, r1, r2, pb, out);
  TORCH_CHECK(!s.f32, "sigmoid_attn_mfma: bf16 only");
  TORCH_CHECK(kafka_hy_sigmoid_attn_mfma_ok(16, (int)s.D, (int)s.Dv, (int)(H / G)), "sigmoid_attn_mfma: sizes");
  TORCH_CHECK(q.stride(0) % 8 == 0 && q_off % 8 == 0 && (reinterpret_cast<uintptr_t>(q.data_ptr()) & 15) == 0,
              "sigmoid_attn_mfma: query rows must be 16-byte aligned");
  TORCH_CHECK(items.is_cuda() && items.scalar_type() == at::kInt && items.is_contiguous() && items.dim() == 2 &&
                  items.size(1) == 4, "sigmoid_attn_mfma: items int32 [n, 4]");
  TORCH_CHECK(tile_tokens >= 1 && tile_tokens * (H / G) <= 32 || (tile_tokens == 1 && H / G <= 32),
              "sigmoid_attn_mfma: a tile holds at most 32 (token, head) rows");
  TORCH_CHECK(t_coef == 0.0 || t_every > 0.0, "sigmoid_attn_mfma: temperature period");
  float* pop = nullptr;
  if (nsplit > 1) {
    TORCH_CHECK(po.has_value() && po->is_cuda() && po->scalar_type() == at::kFloat && po->is_contiguous() &&
                    po->numel() == nsplit * s.T * H * s.Dv, "sigmoid_attn_mfma: po fp32 [nsplit, T, H Dv]");
    pop = po->data_ptr<float>();
  }
  HY_HIP(kafka_hy_sigmoid_attn_mfma(q.data_ptr(), q.stride(0), (int)q_off, kc.data_ptr(), vt.data_ptr(),
                                    bt.data_ptr<int>(), (int)bt.stride(0), items.data_ptr<int>(), (int)items.size(0),
                                    positions.data_ptr<int64_t>(), (int)H, (int)G, (int)s.D, (int)s.Dv, (float)scale,
                                    (float)softcap, (float)t_coef, t_every, r1.data_ptr<float>(),
                                    r2.data_ptr<float>(), pb.data_ptr<float>(), out.data_ptr(), out.stride(0),
                                    (int)nsplit, pop, s.T, stream()));
}

void seg_only(const at::Tensor& seg) {
  TORCH_CHECK(seg.is_cuda() && seg.scalar_type() == at::kInt && seg.is_contiguous() && seg.dim() == 2 &&
                  seg.size(1) == 4, "seg: int32 [R, 4]");
}

void rglru_scan(at::Tensor gates, at::Tensor proj, at::Tensor u, at::Tensor rate, at::Tensor seg, at::Tensor state,
                at::Tensor out, int64_t max_rows) {
  rows2d(gates, "gates"); rows2d(proj, "proj"); rows2d(u, "u"); rows2d(out, "out");
  f32t(gates, "gates"); f32t(rate, "rate"); f32t(state, "state");
  const int f32 = act_f32(u);
  same_act(f32, {&proj, &out});
  const int64_t T = u.size(0), W = u.size(1);
  vec(rate, W, "rate");
  seg_only(seg);
  TORCH_CHECK(gates.size(0) == T && gates.size(1) == 2 * W && proj.size(0) == T && proj.size(1) >= W &&
                  out.size(0) == T && out.size(1) == W, "rglru_scan: shapes");
  TORCH_CHECK(state.is_contiguous() && state.dim() == 2 && state.size(1) == W, "rglru_scan: state fp32 [slots, W]");
  const int64_t R = seg.size(0), CH = kafka_hy_rglru_chunk();
  if (max_rows > CH && R > 0) {
    // long segments: the chunked form (the gates tensor is overwritten with the decays and inputs)
    TORCH_CHECK(max_rows <= T, "rglru_scan: max_rows beyond the step's rows");
    const int64_t nch = (max_rows + CH - 1) / CH;
    auto ab = at::empty({R * nch * 2 * W}, gates.options());
    HY_HIP(kafka_hy_rglru_scan_chunked(f32, gates.data_ptr<float>(), gates.stride(0), proj.data_ptr(), proj.stride(0),
                                       u.data_ptr(), u.stride(0), rate.data_ptr<float>(), seg.data_ptr<int>(), (int)R,
                                       (int)nch, ab.data_ptr<float>(), state.data_ptr<float>(), out.data_ptr(),
                                       out.stride(0), T, (int)W, stream()));
    return;
  }
  HY_HIP(kafka_hy_rglru_scan(f32, gates.data_ptr<float>(), gates.stride(0), proj.data_ptr(), proj.stride(0),
                             u.data_ptr(), u.stride(0), rate.data_ptr<float>(), seg.data_ptr<int>(), (int)seg.size(0),
                             state.data_ptr<float>(), out.data_ptr(), out.stride(0), (int)W, stream()));
}

void mlstm_scan(at::Tensor qkv, at::Tensor gates, int64_t H, int64_t D, int64_t Dv, double cap, at::Tensor seg,
                at::Tensor S, at::Tensor nrm, at::Tensor mx, at::Tensor out) {
  rows2d(qkv, "qkv"); rows2d(gates, "gates"); rows2d(out, "out");
  f32t(gates, "gates"); f32t(S, "S"); f32t(nrm, "n"); f32t(mx, "m"); f32t(out, "out");
  const int f32 = act_f32(qkv);
  const int64_t T = qkv.size(0);
  seg_only(seg);
  TORCH_CHECK(H >= 1 && D >= 1 && Dv >= 1 && D <= kafka_hy_mlstm_max_d(), "mlstm_scan: head sizes (dim up to ",
              kafka_hy_mlstm_max_d(), ")");
  TORCH_CHECK(cap > 0.0, "mlstm_scan: gate cap");
  TORCH_CHECK(qkv.size(1) >= H * (2 * D + Dv) && gates.size(0) == T && gates.size(1) == 2 * H && out.size(0) == T &&
                  out.size(1) == H * Dv, "mlstm_scan: shapes");
  const int64_t slots = S.size(0);
  TORCH_CHECK(S.is_contiguous() && S.dim() == 4 && S.size(1) == H && S.size(2) == D && S.size(3) == Dv &&
                  nrm.is_contiguous() && nrm.dim() == 3 && nrm.size(0) == slots && nrm.size(1) == H &&
                  nrm.size(2) == D && mx.is_contiguous() && mx.dim() == 2 && mx.size(0) == slots && mx.size(1) == H,
              "mlstm_scan: state S [slots, H, D, Dv], n [slots, H, D], m [slots, H]");
  HY_HIP(kafka_hy_mlstm_scan(f32, qkv.data_ptr(), qkv.stride(0), gates.data_ptr<float>(), gates.stride(0), (int)H,
                             (int)D, (int)Dv, (float)cap, seg.data_ptr<int>(), (int)seg.size(0), S.data_ptr<float>(),
                             nrm.data_ptr<float>(), mx.data_ptr<float>(), out.data_ptr<float>(), out.stride(0),
                             stream()));
}

void head_norm_gate(at::Tensor o, at::Tensor w, OptT g, int64_t g_off, int64_t H, double eps, at::Tensor out,
                    double scale) {
  rows2d(o, "o"); rows2d(out, "out"); f32t(o, "o");
  const int f32 = act_f32(out);
  same_act(f32, {&w});
  const int64_t T = o.size(0), n = o.size(1);
  vec(w, n, "w");
  TORCH_CHECK(H >= 1 && n % H == 0 && out.size(0) == T && out.size(1) == n, "head_norm_gate: shapes");
  const void* gp = nullptr; int64_t gs = 0;
  if (g.has_value()) {
    rows2d(*g, "g"); same_act(f32, {&*g});
    TORCH_CHECK(g->size(0) == T && g_off >= 0 && g_off + n <= g->size(1), "head_norm_gate: gate columns");
    gp = g->data_ptr(); gs = g->stride(0);
  }
  HY_HIP(kafka_hy_head_norm_gate(f32, o.data_ptr<float>(), o.stride(0), w.data_ptr(), gp, gs, (int)g_off, (int)H,
                                 (int)(n / H), (float)eps, out.data_ptr(), out.stride(0), T, (float)scale, stream()));
}

void moe_topk(at::Tensor logits, at::Tensor tw, at::Tensor te) {
  rows2d(logits, "logits"); f32t(logits, "logits"); f32t(tw, "weights");
  const int64_t T = logits.size(0), E = logits.size(1);
  TORCH_CHECK(tw.is_contiguous() && tw.dim() == 2 && tw.size(0) == T && te.is_cuda() && te.is_contiguous() &&
                  te.scalar_type() == at::kInt && te.sizes() == tw.sizes(), "moe_topk: outputs [T, k]");
  const int64_t k = tw.size(1);
  TORCH_CHECK(E <= kafka_hy_router_max_e() && k >= 1 && k <= kafka_hy_router_max_k() && k <= E,
              "moe_topk: up to ", kafka_hy_router_max_e(), " experts, ", kafka_hy_router_max_k(), " per row");
  HY_HIP(kafka_hy_moe_topk(logits.data_ptr<float>(), logits.stride(0), (int)E, (int)k, tw.data_ptr<float>(),
                           te.data_ptr<int>(), T, stream()));
}

void moe_rows(at::Tensor h, at::Tensor wgu, at::Tensor wd, at::Tensor tw, at::Tensor te, at::Tensor a, at::Tensor out,
              double limit, double alpha) {
  rows2d(h, "h"); rows2d(out, "out"); f32t(out, "out"); f32t(tw, "weights");
  const int f32 = act_f32(h);
  same_act(f32, {&wgu, &wd, &a});
  const int64_t T = h.size(0), d = h.size(1);
  TORCH_CHECK(wd.is_contiguous() && wd.dim() == 3 && wd.size(1) == d, "moe_rows: w_down [E, d, F]");
  const int64_t E = wd.size(0), F = wd.size(2);
  TORCH_CHECK(wgu.is_contiguous() && wgu.dim() == 3 && wgu.size(0) == E && wgu.size(1) == 2 * F && wgu.size(2) == d,
              "moe_rows: w_gu [E, 2 F, d]");
  TORCH_CHECK(tw.is_contiguous() && tw.dim() == 2 && tw.size(0) == T && te.is_cuda() && te.is_contiguous() &&
                  te.scalar_type() == at::kInt && te.sizes() == tw.sizes(), "moe_rows: routing [T, k]");
  const int64_t k = tw.size(1);
  TORCH_CHECK(a.is_contiguous() && a.numel() == T * k * F, "moe_rows: scratch [T k, F]");
  TORCH_CHECK(out.size(0) == T && out.size(1) == d, "moe_rows: out [T, d]");
  TORCH_CHECK(d <= kafka_hy_moe_rows_max_d() && F <= kafka_hy_moe_rows_max_d(), "moe_rows: row sizes up to ",
              kafka_hy_moe_rows_max_d());
  // expert ids index the weight stacks on the device: the router kernel writes ids in [0, E) only
  HY_HIP(kafka_hy_moe_rows(f32, h.data_ptr(), h.stride(0), wgu.data_ptr(), wd.data_ptr(), tw.data_ptr<float>(),
                           te.data_ptr<int>(), (int)d, (int)F, (int)k, a.data_ptr(), out.data_ptr<float>(),
                           out.stride(0), T, (float)limit, (float)alpha, stream()));
}

void add2(at::Tensor x, at::Tensor y1, OptT y2, OptT w, double eps, OptT out) {
  rows2d(x, "x"); rows2d(y1, "y1"); f32t(x, "x");
  const int f32 = act_f32(y1);
  const int64_t T = x.size(0), d = x.size(1);
  TORCH_CHECK(y1.size(0) == T && y1.size(1) == d, "add2: y1 shape");
  const void* p2 = nullptr; int64_t s2 = 0; int y2f = 0;
  if (y2.has_value()) {
    rows2d(*y2, "y2");
    TORCH_CHECK(y2->size(0) == T && y2->size(1) == d, "add2: y2 shape");
    y2f = y2->scalar_type() == at::kFloat;
    TORCH_CHECK(y2f || act_f32(*y2) == f32, "add2: y2 is fp32 or of y1's dtype");
    p2 = y2->data_ptr(); s2 = y2->stride(0);
  }
  const void* wp = nullptr; void* op = nullptr; int64_t os = 0;
  if (w.has_value()) {
    TORCH_CHECK(out.has_value(), "add2: a norm weight needs an output");
    same_act(f32, {&*w, &*out}); vec(*w, d, "w"); rows2d(*out, "out");
    TORCH_CHECK(out->size(0) == T && out->size(1) == d && x.stride(0) >= d, "add2: out shape");
    wp = w->data_ptr(); op = out->data_ptr(); os = out->stride(0);
  }
  HY_HIP(kafka_hy_add2(f32, x.data_ptr<float>(), x.stride(0), y1.data_ptr(), y1.stride(0), p2, s2, y2f, T, (int)d, wp,
                       (float)eps, op, os, stream()));
}

// ---- residual streams, windowed attention, group-limited router ---------------------------------------------------
const float* f32vec(const OptT& t, int64_t n, const char* name) {
  if (!t.has_value()) return nullptr;
  TORCH_CHECK(t->is_cuda() && t->scalar_type() == at::kFloat && t->is_contiguous() && t->numel() == n, name,
              ": fp32 GPU tensor of ", n, " elements expected");
  return t->data_ptr<float>();
}

void stream_step(at::Tensor xs, OptT y, OptT mix, OptT write, OptT read, OptT norm_w, double eps, OptT out, OptT y2,
                 OptT row_scale, OptT total, bool center) {
  TORCH_CHECK(xs.is_cuda() && xs.scalar_type() == at::kFloat && xs.dim() == 3 && xs.stride(2) == 1,
              "stream_step: streams fp32 [S, T, d] with contiguous rows");
  const int64_t S = xs.size(0), T = xs.size(1), d = xs.size(2);
  TORCH_CHECK(S >= 1 && S <= kafka_hy_stream_max(), "stream_step: 1..", kafka_hy_stream_max(), " streams");
  TORCH_CHECK(T == 0 || (xs.stride(1) >= d && (S == 1 || xs.stride(0) >= d)), "stream_step: overlapping rows");
  TORCH_CHECK(mix.has_value() == write.has_value() && (!mix.has_value() || y.has_value()),
              "stream_step: a write needs mix, write and y");
  TORCH_CHECK(y2.has_value() == row_scale.has_value() && (!y2.has_value() || mix.has_value()),
              "stream_step: y2 and row_scale come together, with a write");
  TORCH_CHECK(read.has_value() == norm_w.has_value() && read.has_value() == out.has_value(),
              "stream_step: a read needs read, norm_w and out");
  const void *yp = nullptr, *y2p = nullptr;
  int64_t ys = 0, y2s = 0;
  int yf = 0, y2f = 0;
  if (mix.has_value()) {
    rows2d(*y, "y");
    TORCH_CHECK(y->size(0) == T && y->size(1) == d, "stream_step: y [T, d]");
    yp = y->data_ptr(); ys = y->stride(0); yf = act_f32(*y);
    if (y2.has_value()) {
      rows2d(*y2, "y2");
      TORCH_CHECK(y2->size(0) == T && y2->size(1) == d, "stream_step: y2 [T, d]");
      y2p = y2->data_ptr(); y2s = y2->stride(0); y2f = act_f32(*y2);
    }
  }
  void* op = nullptr; int64_t os = 0; int of = 0;
  if (out.has_value()) {
    rows2d(*out, "out");
    TORCH_CHECK(out->size(0) == T && out->size(1) == d, "stream_step: out [T, d]");
    op = out->data_ptr(); os = out->stride(0); of = act_f32(*out);
  }
  float* tp = nullptr; int64_t ts = 0;
  if (total.has_value()) {
    rows2d(*total, "total"); f32t(*total, "total");
    TORCH_CHECK(total->size(0) == T && total->size(1) == d, "stream_step: total [T, d]");
    tp = total->data_ptr<float>(); ts = total->stride(0);
  }
  HY_HIP(kafka_hy_stream_step(xs.data_ptr<float>(), xs.stride(0), xs.stride(1), (int)S, yp, ys, yf, y2p, y2s, y2f,
                              f32vec(row_scale, T, "row_scale"), f32vec(mix, S * S, "mix"), f32vec(write, S, "write"),
                              f32vec(read, S, "read"), f32vec(norm_w, d, "norm_w"), (float)eps, op, os, of, tp, ts, T,
                              (int)d, center ? 1 : 0, stream()));
}

void swish_clamp_mul(at::Tensor gu, double limit, double alpha, at::Tensor out) {
  rows2d(gu, "gu"); rows2d(out, "out");
  const int f32 = act_f32(gu);
  same_act(f32, {&out});
  const int64_t T = gu.size(0), F = gu.size(1) / 2;
  TORCH_CHECK(gu.size(1) == 2 * F && out.size(0) == T && out.size(1) == F && limit > 0,
              "swish_clamp_mul: gu [T, 2 F], out [T, F], a positive limit");
  HY_HIP(kafka_hy_swish_clamp_mul(f32, gu.data_ptr(), gu.stride(0), out.data_ptr(), out.stride(0), T, (int)F,
                                  (float)limit, (float)alpha, stream()));
}

void paged_kv(const at::Tensor& kc, const at::Tensor& vt, int64_t Ck, int64_t Cv, const char* who) {
  TORCH_CHECK(kc.is_contiguous() && kc.dim() == 3 && kc.size(1) == 16 && kc.size(2) == Ck && vt.is_contiguous() &&
                  vt.dim() == 3 && vt.size(0) == kc.size(0) && vt.size(1) == Cv && vt.size(2) == 16,
              who, ": keys [pages, 16, G D] and values [pages, G Dv, 16]");
}

void qk_norm_rope_store(at::Tensor qkv, int64_t H, int64_t G, int64_t D, int64_t Dv, at::Tensor qw, at::Tensor kw,
                        double eps, at::Tensor positions, OptT cos_sin, int64_t dims, OptT v_first,
                        int64_t v_first_off, double lam, at::Tensor kc, at::Tensor vt, at::Tensor slots,
                        at::Tensor q_out) {
  rows2d(qkv, "qkv"); rows2d(q_out, "q_out");
  const int f32 = act_f32(qkv);
  same_act(f32, {&kc, &vt, &q_out});
  const int64_t T = qkv.size(0);
  TORCH_CHECK(H > 0 && G > 0 && H % G == 0 && D > 0 && Dv > 0 && qkv.size(1) >= H * D + G * D + G * Dv &&
                  q_out.size(0) == T && q_out.size(1) == H * D, "qk_norm_rope_store: head sizes");
  TORCH_CHECK(dims >= 0 && dims % 2 == 0 && dims <= D && cos_sin.has_value() == (dims > 0),
              "qk_norm_rope_store: rot dims even, at most the head size, with their table");
  TORCH_CHECK(positions.is_cuda() && positions.scalar_type() == at::kLong && positions.is_contiguous() &&
                  positions.numel() == T && slots.is_cuda() && slots.scalar_type() == at::kLong &&
                  slots.is_contiguous() && slots.numel() == T, "qk_norm_rope_store: positions / slots int64 [T]");
  if (dims > 0)
    TORCH_CHECK(cos_sin->is_cuda() && cos_sin->scalar_type() == at::kFloat && cos_sin->is_contiguous() &&
                    cos_sin->dim() == 2 && cos_sin->size(1) == dims, "qk_norm_rope_store: cos_sin fp32 [positions, dims]");
  paged_kv(kc, vt, G * D, G * Dv, "qk_norm_rope_store");
  const void* vfp = nullptr; int64_t vfs = 0;
  if (v_first.has_value()) {
    rows2d(*v_first, "v_first"); same_act(f32, {&*v_first});
    TORCH_CHECK(v_first->size(0) == T && v_first_off >= 0 && v_first_off + G * Dv <= v_first->size(1),
                "qk_norm_rope_store: the earlier layer's value columns");
    vfp = v_first->data_ptr(); vfs = v_first->stride(0);
  }
  // positions index the table's rows and slots the cache on the device: the step plan keeps both in range
  HY_HIP(kafka_hy_qk_norm_rope_store(f32, qkv.data_ptr(), qkv.stride(0), (int)H, (int)G, (int)D, (int)Dv,
                                     f32vec(qw, H * D, "q norm weight"), f32vec(kw, G * D, "k norm weight"), (float)eps,
                                     positions.data_ptr<int64_t>(), dims > 0 ? cos_sin->data_ptr<float>() : nullptr,
                                     (int)dims, vfp, vfs, (int)v_first_off, (float)lam, kc.data_ptr(), vt.data_ptr(),
                                     slots.data_ptr<int64_t>(), q_out.data_ptr(), q_out.stride(0), T, stream()));
}

void window_attn(at::Tensor q, at::Tensor kc, at::Tensor vt, at::Tensor bt, at::Tensor tok_seg, at::Tensor positions,
                 int64_t H, int64_t G, double scale, int64_t window, OptT sink, at::Tensor out, bool shared_keys) {
  rows2d(q, "q"); rows2d(out, "out");
  const int f32 = act_f32(q);
  same_act(f32, {&kc, &vt, &out});
  const int64_t T = q.size(0);
  TORCH_CHECK(H > 0 && G > 0 && H % G == 0 && q.size(1) % H == 0 && out.size(0) == T && out.size(1) % H == 0,
              "window_attn: heads");
  // shared_keys: a query row has the whole key row's size and meets all G key heads of a token
  const int64_t D = q.size(1) / H, Dv = out.size(1) / H;
  paged_kv(kc, vt, shared_keys ? D : G * D, G * Dv, "window_attn");
  TORCH_CHECK(D <= kafka_hy_window_attn_max_d() && Dv <= kafka_hy_window_attn_max_dv(), "window_attn: head sizes up to ",
              kafka_hy_window_attn_max_d(), " / ", kafka_hy_window_attn_max_dv());
  TORCH_CHECK(window >= 0, "window_attn: window");
  TORCH_CHECK(bt.is_cuda() && bt.scalar_type() == at::kInt && bt.dim() == 2 && bt.stride(1) == 1 &&
                  tok_seg.is_cuda() && tok_seg.scalar_type() == at::kInt && tok_seg.is_contiguous() &&
                  tok_seg.numel() == T && positions.is_cuda() && positions.scalar_type() == at::kLong &&
                  positions.is_contiguous() && positions.numel() == T, "window_attn: block tables / tok_seg / positions");
  HY_HIP(kafka_hy_window_attn(f32, q.data_ptr(), q.stride(0), kc.data_ptr(), vt.data_ptr(), bt.data_ptr<int>(),
                              (int)bt.stride(0), tok_seg.data_ptr<int>(), positions.data_ptr<int64_t>(), (int)H, (int)G,
                              (int)D, (int)Dv, (float)scale, (int)window, sink_ptr(sink, H), out.data_ptr(),
                              out.stride(0), T, shared_keys ? 1 : 0, stream()));
}

// the matrix-core kernel: items int32 [n, 4] = (first row, tokens, segment, 0), each at most 32 (token, query head of
// one key/value head) rows of one segment
void window_attn_mfma(at::Tensor q, at::Tensor kc, at::Tensor vt, at::Tensor bt, at::Tensor items, int64_t tile_tokens,
                      at::Tensor positions, int64_t H, int64_t G, double scale, int64_t window, OptT sink,
                      at::Tensor out, int64_t nsplit, OptT po, OptT pml, bool shared_keys) {
  for (const at::Tensor* t : {&q, &kc, &vt, &out})
    TORCH_CHECK(t->is_cuda() && t->scalar_type() == at::kBFloat16, "window_attn_mfma: bf16 GPU tensors");
  rows2d(q, "q"); rows2d(out, "out");
  const int64_t T = q.size(0);
  TORCH_CHECK(H > 0 && G > 0 && H % G == 0 && q.size(1) % H == 0 && out.size(0) == T && out.size(1) % H == 0,
              "window_attn_mfma: heads");
  const int64_t D = q.size(1) / H, Dv = out.size(1) / H, rep = H / G;
  paged_kv(kc, vt, shared_keys ? D : G * D, G * Dv, "window_attn_mfma");
  TORCH_CHECK(kafka_hy_window_attn_mfma_ok(16, (int)D, (int)Dv, (int)rep), "window_attn_mfma: sizes not supported");
  // 16-byte loads: every query row start must be a multiple of 8 elements
  TORCH_CHECK(q.stride(0) % 8 == 0 && (reinterpret_cast<uintptr_t>(q.data_ptr()) & 15) == 0,
              "window_attn_mfma: query alignment");
  TORCH_CHECK(tile_tokens >= 1 && tile_tokens * rep <= 32, "window_attn_mfma: a tile holds at most 32 rows");
  TORCH_CHECK(window >= 0, "window_attn_mfma: window");
  TORCH_CHECK(bt.is_cuda() && bt.scalar_type() == at::kInt && bt.dim() == 2 && bt.stride(1) == 1 && items.is_cuda() &&
                  items.scalar_type() == at::kInt && items.is_contiguous() && items.dim() == 2 && items.size(1) == 4 &&
                  positions.is_cuda() && positions.scalar_type() == at::kLong && positions.is_contiguous() &&
                  positions.numel() == T, "window_attn_mfma: block tables / items / positions");
  float *pop = nullptr, *pmlp = nullptr;
  TORCH_CHECK(nsplit >= 1 && nsplit <= 64, "window_attn_mfma: 1..64 key-range splits");
  if (nsplit > 1) {
    TORCH_CHECK(po.has_value() && pml.has_value() && po->is_cuda() && po->scalar_type() == at::kFloat &&
                    po->is_contiguous() && po->numel() >= nsplit * T * H * Dv && pml->is_cuda() &&
                    pml->scalar_type() == at::kFloat && pml->is_contiguous() && pml->numel() >= nsplit * T * H * 2,
                "window_attn_mfma: split workspaces fp32 [splits, T, H Dv] and [splits, T, H, 2]");
    pop = po->data_ptr<float>(); pmlp = pml->data_ptr<float>();
  }
  // the tiles' rows, tokens and segments come from the step plan, which keeps them inside the step
  HY_HIP(kafka_hy_window_attn_mfma(q.data_ptr(), q.stride(0), kc.data_ptr(), vt.data_ptr(), bt.data_ptr<int>(),
                                   (int)bt.stride(0), items.data_ptr<int>(), (int)items.size(0),
                                   positions.data_ptr<int64_t>(), (int)H, (int)G, (int)D, (int)Dv, (float)scale,
                                   (int)window, sink_ptr(sink, H), out.data_ptr(), out.stride(0), (int)nsplit, pop,
                                   pmlp, T, shared_keys ? 1 : 0, stream()));
}

void moe_topk_grouped(at::Tensor logits, int64_t E, at::Tensor corr, int64_t groups, int64_t keep, double eps,
                      at::Tensor tw, at::Tensor te, OptT gate) {
  rows2d(logits, "logits"); f32t(logits, "logits"); f32t(tw, "weights");
  const int64_t T = logits.size(0);
  TORCH_CHECK(tw.is_contiguous() && tw.dim() == 2 && tw.size(0) == T && te.is_cuda() && te.is_contiguous() &&
                  te.scalar_type() == at::kInt && te.sizes() == tw.sizes(), "moe_topk_grouped: outputs [T, k]");
  const int64_t k = tw.size(1);
  TORCH_CHECK(E >= 1 && E + (gate.has_value() ? 1 : 0) <= logits.size(1) && E <= kafka_hy_grouped_router_max_e() &&
                  k >= 1 && k <= kafka_hy_grouped_router_max_k() && groups >= 1 &&
                  groups <= kafka_hy_grouped_router_max_g() && E % groups == 0 && keep >= 1 && keep <= groups &&
                  k <= keep * (E / groups),
              "moe_topk_grouped: up to ", kafka_hy_grouped_router_max_e(), " experts in up to ",
              kafka_hy_grouped_router_max_g(), " equal groups, ", kafka_hy_grouped_router_max_k(),
              " per row within the kept groups");
  HY_HIP(kafka_hy_moe_topk_grouped(logits.data_ptr<float>(), logits.stride(0), (int)E, (int)k,
                                   f32vec(corr, E, "correction"), (int)groups, (int)keep, (float)eps,
                                   tw.data_ptr<float>(), te.data_ptr<int>(),
                                   const_cast<float*>(f32vec(gate, T, "gate")), T, stream()));
}

void act_norm(at::Tensor x, int64_t c0, int64_t n, at::Tensor w, double eps, at::Tensor out, bool center) {
  rows2d(x, "x"); rows2d(out, "out"); f32t(w, "w");
  const int f32 = act_f32(x);
  same_act(f32, {&out});
  const int64_t T = x.size(0);
  vec(w, n, "w");
  TORCH_CHECK(c0 >= 0 && n >= 1 && c0 + n <= x.size(1) && out.size(0) == T && out.size(1) == n, "act_norm: columns");
  HY_HIP(kafka_hy_act_norm(f32, x.data_ptr(), x.stride(0), (int)c0, (int)n, w.data_ptr<float>(), (float)eps,
                           out.data_ptr(), out.stride(0), T, center ? 1 : 0, stream()));
}

void gate_mul(at::Tensor a, at::Tensor g, int64_t g_off, double scale, at::Tensor out) {
  rows2d(a, "a"); rows2d(g, "g"); rows2d(out, "out");
  const int f32 = act_f32(a);
  same_act(f32, {&g, &out});
  const int64_t T = a.size(0), n = a.size(1);
  TORCH_CHECK(g.size(0) == T && g_off >= 0 && g_off + n <= g.size(1) && out.size(0) == T && out.size(1) == n,
              "gate_mul: shapes");
  HY_HIP(kafka_hy_gate_mul(f32, a.data_ptr(), a.stride(0), g.data_ptr(), g.stride(0), (int)g_off, (float)scale,
                           out.data_ptr(), out.stride(0), T, (int)n, stream()));
}

// (seg comes from the step plan, which keeps every segment's rows inside the step)
void mingru_scan(at::Tensor proj, at::Tensor bias, int64_t W, at::Tensor seg, at::Tensor state, at::Tensor out,
                 int64_t max_rows) {
  rows2d(proj, "proj"); rows2d(out, "out"); f32t(bias, "bias"); f32t(state, "state");
  const int f32 = act_f32(proj);
  same_act(f32, {&out});
  const int64_t T = proj.size(0);
  seg_only(seg);
  TORCH_CHECK(W >= 1 && proj.size(1) >= 3 * W && out.size(0) == T && out.size(1) == W, "mingru_scan: shapes");
  vec(bias, 2 * W, "bias");
  TORCH_CHECK(state.is_contiguous() && state.dim() == 2 && state.size(1) == W, "mingru_scan: state fp32 [slots, W]");
  const int64_t R = seg.size(0), CH = kafka_hy_mingru_chunk();
  if (max_rows > CH && R > 0) {
    TORCH_CHECK(max_rows <= T, "mingru_scan: max_rows beyond the step's rows");
    const int64_t nch = (max_rows + CH - 1) / CH;
    auto ab = at::empty({T * 2 * W}, state.options());
    auto ce = at::empty({R * nch * 2 * W}, state.options());
    HY_HIP(kafka_hy_mingru_scan_chunked(f32, proj.data_ptr(), proj.stride(0), bias.data_ptr<float>(),
                                        seg.data_ptr<int>(), (int)R, (int)nch, ab.data_ptr<float>(),
                                        ce.data_ptr<float>(), state.data_ptr<float>(), out.data_ptr(), out.stride(0), T,
                                        (int)W, stream()));
    return;
  }
  HY_HIP(kafka_hy_mingru_scan(f32, proj.data_ptr(), proj.stride(0), bias.data_ptr<float>(), seg.data_ptr<int>(), (int)R,
                              state.data_ptr<float>(), out.data_ptr(), out.stride(0), (int)W, stream()));
}

void hgrn2_scan(at::Tensor proj, int64_t q_off, int64_t f_off, int64_t v_off, at::Tensor f_bias, at::Tensor lower,
                int64_t H, int64_t D, int64_t Dv, at::Tensor seg, at::Tensor S, at::Tensor out) {
  rows2d(proj, "proj"); rows2d(out, "out"); f32t(f_bias, "f_bias"); f32t(lower, "lower"); f32t(S, "S"); f32t(out, "out");
  const int f32 = act_f32(proj);
  const int64_t T = proj.size(0), C = proj.size(1);
  seg_only(seg);
  TORCH_CHECK(H >= 1 && D >= 1 && Dv >= 1 && D <= kafka_hy_hgrn2_max_d(), "hgrn2_scan: head sizes (dim up to ",
              kafka_hy_hgrn2_max_d(), ")");
  TORCH_CHECK(q_off >= 0 && q_off + H * D <= C && f_off >= 0 && f_off + H * D <= C && v_off >= 0 &&
                  v_off + H * Dv <= C && out.size(0) == T && out.size(1) == H * Dv, "hgrn2_scan: columns");
  vec(f_bias, H * D, "f_bias"); vec(lower, H * D, "lower");
  TORCH_CHECK(S.is_contiguous() && S.dim() == 4 && S.size(1) == H && S.size(2) == D && S.size(3) == Dv,
              "hgrn2_scan: state fp32 [slots, H, D, Dv]");
  HY_HIP(kafka_hy_hgrn2_scan(f32, proj.data_ptr(), proj.stride(0), (int)q_off, (int)f_off, (int)v_off,
                             f_bias.data_ptr<float>(), lower.data_ptr<float>(), (int)H, (int)D, (int)Dv,
                             seg.data_ptr<int>(), (int)seg.size(0), S.data_ptr<float>(), out.data_ptr<float>(),
                             out.stride(0), stream()));
}

void rope_kv_store(at::Tensor qkv, int64_t H, int64_t G, int64_t D, int64_t Dv, at::Tensor positions, OptT cos_sin,
                   int64_t dims, bool pairs, OptT talk, at::Tensor kc, at::Tensor vt, at::Tensor slots,
                   at::Tensor q_out) {
  rows2d(qkv, "qkv"); rows2d(q_out, "q_out");
  const int f32 = act_f32(qkv);
  same_act(f32, {&kc, &vt, &q_out});
  const int64_t T = qkv.size(0);
  TORCH_CHECK(H > 0 && G > 0 && H % G == 0 && D > 0 && Dv > 0 && qkv.size(1) >= H * D + G * D + G * Dv &&
                  q_out.size(0) == T && q_out.size(1) == (talk.has_value() ? H * G * D : H * D),
              "rope_kv_store: head sizes (q_out [T, H D], or [T, H G D] with a head mix)");
  TORCH_CHECK(dims >= 0 && dims % 2 == 0 && dims <= D && cos_sin.has_value() == (dims > 0),
              "rope_kv_store: rot dims even, at most the head size, with their table");
  TORCH_CHECK(positions.is_cuda() && positions.scalar_type() == at::kLong && positions.is_contiguous() &&
                  positions.numel() == T && slots.is_cuda() && slots.scalar_type() == at::kLong &&
                  slots.is_contiguous() && slots.numel() == T, "rope_kv_store: positions / slots int64 [T]");
  if (dims > 0)
    TORCH_CHECK(cos_sin->is_cuda() && cos_sin->scalar_type() == at::kFloat && cos_sin->is_contiguous() &&
                    cos_sin->dim() == 2 && cos_sin->size(1) == dims, "rope_kv_store: cos_sin fp32 [positions, dims]");
  TORCH_CHECK((H + G) * D + dims + (talk.has_value() ? H * H : 0) <= kafka_hy_rope_store_max_q(),
              "rope_kv_store: q and k of a row, the rotation's table row and the head mix must fit ",
              kafka_hy_rope_store_max_q(), " floats");
  paged_kv(kc, vt, G * D, G * Dv, "rope_kv_store");
  // positions index the table's rows and slots the cache on the device: the step plan keeps both in range
  HY_HIP(kafka_hy_rope_kv_store(f32, qkv.data_ptr(), qkv.stride(0), (int)H, (int)G, (int)D, (int)Dv,
                                positions.data_ptr<int64_t>(), dims > 0 ? cos_sin->data_ptr<float>() : nullptr,
                                (int)dims, pairs ? 1 : 0, f32vec(talk, H * H, "head mix"), kc.data_ptr(), vt.data_ptr(),
                                slots.data_ptr<int64_t>(), q_out.data_ptr(), q_out.stride(0), T, stream()));
}

// the chunk tables come from ops.hybrid.scan_chunks, which keeps chunks inside their segments and numbers them 0 .. n - 1
void hgrn2_chunk_decay(at::Tensor proj, int64_t f_off, at::Tensor f_bias, at::Tensor lower, at::Tensor vseg,
                       at::Tensor F) {
  rows2d(proj, "proj"); f32t(f_bias, "f_bias"); f32t(lower, "lower"); f32t(F, "F");
  seg_only(vseg);
  const int64_t HD = lower.numel();
  vec(f_bias, HD, "f_bias");
  TORCH_CHECK(lower.is_contiguous() && f_off >= 0 && f_off + HD <= proj.size(1) && F.is_contiguous() &&
                  F.numel() == vseg.size(0) * HD, "hgrn2_chunk_decay: shapes");
  HY_HIP(kafka_hy_hgrn2_decay(act_f32(proj), proj.data_ptr(), proj.stride(0), (int)f_off, f_bias.data_ptr<float>(),
                              lower.data_ptr<float>(), (int)HD, vseg.data_ptr<int>(), (int)vseg.size(0),
                              F.data_ptr<float>(), stream()));
}

void hgrn2_chunk_combine(at::Tensor cs, at::Tensor F, at::Tensor tmp, at::Tensor state) {
  seg_only(cs); f32t(F, "F"); f32t(tmp, "tmp"); f32t(state, "state");
  TORCH_CHECK(tmp.is_contiguous() && tmp.dim() == 4 && state.is_contiguous() && state.dim() == 4 &&
                  tmp.size(1) == state.size(1) && tmp.size(2) == state.size(2) && tmp.size(3) == state.size(3) &&
                  F.is_contiguous() && F.numel() == tmp.size(0) * tmp.size(1) * tmp.size(2),
              "hgrn2_chunk_combine: tmp [chunks, H, D, Dv], state [slots, H, D, Dv], F [chunks, H D]");
  HY_HIP(kafka_hy_hgrn2_combine(cs.data_ptr<int>(), (int)cs.size(0), F.data_ptr<float>(),
                                (int)(tmp.size(1) * tmp.size(2)), (int)tmp.size(3), tmp.data_ptr<float>(),
                                state.data_ptr<float>(), stream()));
}

}  // namespace


void kafka_bind_hybrid(pybind11::module_& m) {
  namespace py = pybind11;
  m.def("hy_ln_shift", &ln_shift, py::arg("x"), py::arg("w"), py::arg("b"), py::arg("eps"), py::arg("out"),
        py::arg("mu") = py::none(), py::arg("tok_seg") = py::none(), py::arg("seg") = py::none(),
        py::arg("state") = py::none(), py::arg("last") = py::none());
  m.def("hy_scatter_rows", &scatter_rows);
  m.def("hy_add_ln", &add_ln, py::arg("x"), py::arg("y"), py::arg("w"), py::arg("b"), py::arg("eps"),
        py::arg("out2") = py::none(), py::arg("w2") = py::none(), py::arg("b2") = py::none());
  m.def("hy_gelu_mul", &gelu_mul);
  m.def("hy_side_gate", &side_gate);
  m.def("hy_side_dwa", &side_dwa);
  m.def("hy_latent_prep", &latent_prep, py::arg("qgd"), py::arg("H"), py::arg("dim"), py::arg("rd"), py::arg("R"),
        py::arg("dkv_off"), py::arg("dkv_w"), py::arg("eps"), py::arg("positions"), py::arg("cos_sin"),
        py::arg("dims"), py::arg("cache"), py::arg("slots"), py::arg("q_rot"), py::arg("cache_t") = py::none());
  m.def("hy_latent_attn_mfma", &latent_attn_mfma, py::arg("q_lat"), py::arg("q_rot"), py::arg("cache"),
        py::arg("cache_t"), py::arg("bt"), py::arg("items"), py::arg("tile_tokens"), py::arg("positions"),
        py::arg("scale"), py::arg("out"), py::arg("nsplit") = 1, py::arg("po") = py::none(),
        py::arg("pml") = py::none(), py::arg("window") = 0, py::arg("sink") = py::none());
  m.def("hy_latent_mfma_ok", [](int page, int R, int rd) { return kafka_hy_latent_mfma_ok(page, R, rd) != 0; });
  m.def("hy_sigmoid_mul", &sigmoid_mul);
  m.def("hy_latent_attn", &latent_attn, py::arg("q_lat"), py::arg("q_rot"), py::arg("cache"), py::arg("bt"),
        py::arg("tok_seg"), py::arg("positions"), py::arg("scale"), py::arg("out"), py::arg("window") = 0,
        py::arg("sink") = py::none());
  m.def("hy_short_conv", &short_conv);
  m.def("hy_ssm_scan", &ssm_scan);
  m.def("hy_ssm_combine", &ssm_combine);
  m.def("hy_gated_norm", &gated_norm);
  m.def("hy_scan_groups", [](int P, int N) { return kafka_hy_scan_groups(P, N); });
  m.def("hy_rms_norm", &rms_norm);
  m.def("hy_kv_store", &kv_store);
  m.def("hy_sigmoid_attn", &sigmoid_attn);
  m.def("hy_rglru_scan", &rglru_scan, py::arg("gates"), py::arg("proj"), py::arg("u"), py::arg("rate"), py::arg("seg"),
        py::arg("state"), py::arg("out"), py::arg("max_rows") = 0);
  m.def("hy_mlstm_scan", &mlstm_scan);
  m.def("hy_head_norm_gate", &head_norm_gate, py::arg("o"), py::arg("w"), py::arg("g"), py::arg("g_off"), py::arg("H"),
        py::arg("eps"), py::arg("out"), py::arg("scale") = 1.0);
  m.def("hy_moe_topk", &moe_topk);
  m.def("hy_moe_rows", &moe_rows, py::arg("h"), py::arg("wgu"), py::arg("wd"), py::arg("tw"), py::arg("te"),
        py::arg("a"), py::arg("out"), py::arg("limit") = 0.0, py::arg("alpha") = 1.0);
  m.def("hy_add2", &add2, py::arg("x"), py::arg("y1"), py::arg("y2") = py::none(), py::arg("w") = py::none(),
        py::arg("eps") = 0.0, py::arg("out") = py::none());
  m.def("hy_stream_step", &stream_step, py::arg("xs"), py::arg("y") = py::none(), py::arg("mix") = py::none(),
        py::arg("write") = py::none(), py::arg("read") = py::none(), py::arg("norm_w") = py::none(),
        py::arg("eps") = 0.0, py::arg("out") = py::none(), py::arg("y2") = py::none(),
        py::arg("row_scale") = py::none(), py::arg("total") = py::none(), py::arg("center") = false);
  m.def("hy_swish_clamp_mul", &swish_clamp_mul);
  m.def("hy_qk_norm_rope_store", &qk_norm_rope_store);
  m.def("hy_window_attn", &window_attn, py::arg("q"), py::arg("kc"), py::arg("vt"), py::arg("bt"), py::arg("tok_seg"),
        py::arg("positions"), py::arg("H"), py::arg("G"), py::arg("scale"), py::arg("window"), py::arg("sink"),
        py::arg("out"), py::arg("shared_keys") = false);
  m.def("hy_window_attn_mfma_ok",
        [](int page, int D, int Dv, int rep) { return kafka_hy_window_attn_mfma_ok(page, D, Dv, rep) != 0; });
  m.def("hy_window_attn_mfma", &window_attn_mfma, py::arg("q"), py::arg("kc"), py::arg("vt"), py::arg("bt"),
        py::arg("items"), py::arg("tile_tokens"), py::arg("positions"), py::arg("H"), py::arg("G"), py::arg("scale"),
        py::arg("window"), py::arg("sink"), py::arg("out"), py::arg("nsplit") = 1, py::arg("po") = py::none(),
        py::arg("pml") = py::none(), py::arg("shared_keys") = false);
  m.def("hy_moe_topk_grouped", &moe_topk_grouped);
  m.def("hy_act_norm", &act_norm);
  m.def("hy_gate_mul", &gate_mul);
  m.def("hy_mingru_scan", &mingru_scan, py::arg("proj"), py::arg("bias"), py::arg("W"), py::arg("seg"),
        py::arg("state"), py::arg("out"), py::arg("max_rows") = 0);
  m.def("hy_hgrn2_scan", &hgrn2_scan);
  m.def("hy_hgrn2_chunk_decay", &hgrn2_chunk_decay);
  m.def("hy_hgrn2_chunk_combine", &hgrn2_chunk_combine);
  m.def("hy_rope_kv_store", &rope_kv_store);
  m.def("hy_sigmoid_attn_mfma_ok",
        [](int page, int D, int Dv, int rep) { return kafka_hy_sigmoid_attn_mfma_ok(page, D, Dv, rep) != 0; });
  m.def("hy_sigmoid_attn_mfma", &sigmoid_attn_mfma, py::arg("q"), py::arg("q_off"), py::arg("kc"), py::arg("vt"),
        py::arg("bt"), py::arg("items"), py::arg("tile_tokens"), py::arg("positions"), py::arg("H"), py::arg("G"),
        py::arg("scale"), py::arg("softcap"), py::arg("t_coef"), py::arg("t_every"), py::arg("r1"), py::arg("r2"),
        py::arg("pb"), py::arg("out"), py::arg("nsplit") = 1, py::arg("po") = py::none());
}
