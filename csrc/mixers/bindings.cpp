// PyTorch bindings of the sequence-mixer / MoE kernels (extension `_C_mixers`).
//
// As in csrc/bindings.cpp every op validates dtype / device / shape on the host (a
// mis-shaped launch of a hand-written kernel can fault the GPU) and launches on the
// caller's current stream without allocating or synchronising.
#include <algorithm>

#include <torch/extension.h>
#include <c10/hip/HIPStream.h>
#include <hip/hip_runtime.h>

extern "C" {
int mx_embed_rows(float* out, const int* ids, const void* table, int bf16, int rows, int width, int vocab,
                  float scale, const int* positions, const float* freqs, hipStream_t s);
int mx_layer_norm(float* x, const void* y, int y_bf16, long y_stride, const float* w, const float* b, void* out,
                  void* cast, int out_bf16, int rows, int width, float eps, hipStream_t s);
int mx_tanh_cap(float* x, long n, float cap, hipStream_t s);
int mx_grouped_gemm(void* C, const void* A, const void* W, const int* offs, int groups, long M, int N, int K,
                    hipStream_t s);
int mx_relu_sq_rows(void* out, const void* u, int bf16, long u_stride, long rows, int ff, hipStream_t s);
int mx_gather_add_rows(float* out, const void* y, int y_bf16, const int* idx, const float* w, long rows, int top,
                       int width, long y_rows, hipStream_t s);
int mx_conv_attn_prep(float* q_out, const void* qkv, int bf16, long stride, int nq, int nk, int nv,
                      const float* conv_w, int taps, float* hist, const int* start, const int* pos0, const int* slot,
                      int num_segs, int num_state_slots, const float* wq, const float* wk, float eps, int head_dim,
                      const int* slots, void* k_cache, void* v_cache, int cache_bf16, long num_slots, long rows,
                      hipStream_t s);
int mx_moe_top_logits(int* idx, float* wts, const float* z, long rows, int experts, int top, hipStream_t s);
int mx_moe_route_top_logits(int* idx, float* wts, const void* h, int bf16, long h_stride, const float* router,
                            const float* bias, long rows, int experts, int width, int top, hipStream_t s);
int mx_gelu_glu(void* out, const void* gu, int bf16, long gu_stride, long rows, int ff, int relu, hipStream_t s);
int mx_gla_max_dk();
int mx_gla_scan(float* o, const void* qkv, int bf16, long qkv_stride, const void* a, long a_stride,
                const float* a_bias, float tau, float* state, const int* start, const int* pos0, const int* slot,
                int num_segs, int max_rows, int heads, int dk, int dv, int num_slots, hipStream_t s);
int mx_pair_embed_add(float* x, const int* ids, const void* table, int bf16, int rows, int width, long mul_prev,
                      long mul_cur, int buckets, const int* start, const int* pos0, const int* slot, int num_segs,
                      int* last_tok, int num_slots, const void* embed, int vocab, float scale, hipStream_t s);
int mx_add_scaled_rms_norm(float* x, const void* y1, int y1_bf16, long y1_stride, const void* y2, int y2_bf16,
                           long y2_stride, float mult, const float* next_w, void* out, int out_bf16, int rows,
                           int width, float eps, hipStream_t s);
int mx_dual_rms_mean(float* out, const void* a, long a_stride, const void* b, long b_stride, int bf16,
                     const float* wa, const float* wb, int rows, int width, float eps, float scale, hipStream_t s);
int mx_sigmoid_gate(void* out, int out_bf16, const float* o, const void* g, int g_bf16, long g_stride, long rows,
                    int n, hipStream_t s);
int mx_attn_prep(float* q_out, const void* qkv, int bf16, long stride, int nq, int nk, int nv, const float* wq,
                 const float* wk, float eps, const float* table, int table_rows, int rot_dims, int head_dim,
                 const int* positions, const int* slots, void* k_cache, void* v_cache, int cache_bf16,
                 long num_slots, long rows, hipStream_t s);
int mx_window_max_dv();
int mx_window_attention(float* out, const float* q, const void* k_cache, const void* v_cache, int cache_bf16,
                        const int* start, const int* pos0, const int* kv_len, const int* bt, int bt_stride,
                        int num_segs, long total_rows, int heads, int maps, int kv_heads, int dk, int dv, int window,
                        float scale, int sigmoid, const float* r1, const float* r2, const float* pb, int block_size,
                        int num_blocks, int skip_from, float softcap, int has_sink, float sink, int blocks,
                        int keep_first, const float* dist_bias, int nd, hipStream_t s);
int mx_band_weights(float* S, int gk, int rep_rows_total, int rows, int keys, int first_pos, int key0, int heads,
                    int maps, int kv_heads, int window, float scale, int sigmoid, const float* r1, const float* r2,
                    const float* pb, float softcap, int has_sink, float sink, int blocks, int keep_first, int ext,
                    const float* dist_bias, int nd, hipStream_t s);
int mx_diff_combine(void* out, int out_bf16, const float* a, const void* gate, int gate_bf16, long gate_stride,
                    long rows, int heads, int dv, float lam, float post, float eps, hipStream_t s);
int mx_ssd_max_state();
int mx_ssd_scan(float* y, const void* xbc, int bf16, long x_stride, const void* dt, long dt_stride,
                const float* a_log, const float* dt_bias, const float* d_skip, float* state, const int* start,
                const int* pos0, const int* slot, int num_segs, int heads, int groups, int n, int dv, int num_slots,
                hipStream_t s);
int mx_gate_group_norm(void* out, int out_bf16, const float* y, const void* z, int z_bf16, long z_stride,
                       const float* w, long rows, int groups, int gs, float eps, hipStream_t s);
int mx_add_rms_norm(float* x, const void* y, int y_bf16, long y_stride, const float* wb, const float* add_vec,
                    const float* next_w, void* out, void* cast, int out_bf16, int rows, int width, float eps,
                    hipStream_t s);
int mx_head_rms_gate(void* out, int out_bf16, const float* o, const float* w, const void* gate, int gate_bf16,
                     long gate_stride, long rows, int heads, int dv, float eps, int silu, hipStream_t s);
int mx_relu_sq(void* x, int bf16, long n, hipStream_t s);
int mx_clamp_swiglu(void* out, const void* gu, int bf16, long gu_stride, long rows, int ff, float limit,
                    hipStream_t s);
int mx_side_gate(void* out, const void* gpre, const void* table, int bf16, long table_stride, const int* ids,
                 int col0, long rows, int sd, int vocab, hipStream_t s);
int mx_scale_add_rows(float* out, const void* y, int y_bf16, const int* rows, const void* weights, int w_bf16,
                      int sigmoid, long n, int width, int out_rows, hipStream_t s);
int mx_short_conv_silu(void* out, const void* x, int bf16, long x_stride, const float* w, const float* bias,
                       float* hist, const int* start, const int* pos0, const int* slot, int num_segs, int max_rows,
                       int channels, int taps, int num_slots, hipStream_t s);
int mx_delta_prep(float* qn, float* kn, float* g, float* beta, const void* qkv, int bf16, long qkv_stride,
                  const void* a, long a_stride, const void* b, long b_stride, const float* a_log,
                  const float* dt_bias, long rows, int heads, int kv_heads, int dk, hipStream_t s);
int mx_delta_max_dk();
int mx_delta_rule(float* o, const float* qn, const float* kn, const float* g, const float* beta,
                  const void* qkv, int bf16, long qkv_stride, float* state, const int* start, const int* pos0,
                  const int* slot, int num_segs, int heads, int kv_heads, int dk, int dv, int num_slots,
                  hipStream_t s);
int mx_latent_kv_write(const void* dkv, int bf16, long stride, const float* w, float eps, const float* table,
                       int table_rows, int dims, const int* positions, const int* slots, void* cache,
                       int cache_bf16, long num_slots, long rows, int rank, int dr, hipStream_t s);
int mx_latent_q_rope(float* qn, float* qr, const void* q, int bf16, long stride, const float* table,
                     int table_rows, int dims, const int* positions, long rows, int heads, int dn, int dr,
                     hipStream_t s);
int mx_latent_max_rank();
int mx_latent_attention(float* out, const float* qa, const float* qr, const void* cache, int cache_bf16,
                        const int* start, const int* pos0, const int* kv_len, const int* bt, int bt_stride,
                        int num_segs, int max_rows, int heads, long total_rows, int rank, int dr,
                        int block_size, int num_blocks, float scale, int skip_from, hipStream_t s);
long mx_latent_split_ws(int heads, int rank, int dr);
int mx_latent_attention_split(float* out, float* ws_acc, float* ws_ml, const float* qa, const float* qr,
                              const void* cache, int cache_bf16, const int* start, const int* pos0,
                              const int* kv_len, const int* bt, int bt_stride, int num_segs, int max_rows,
                              int heads, long total_rows, int rank, int dr, int block_size, int num_blocks,
                              float scale, int skip_from, int splits, hipStream_t s);
int mx_causal_softmax(void* P, int p_bf16, const float* S, long rows, int rows_per_head, int first_pos, int ncols,
                      float scale, hipStream_t s);
int mx_moe_pairs(float* out, void* y, const void* h, int bf16, long h_stride, const int* idx, const float* wts,
                 const void* wgu, const void* wdown, long rows, int top, int experts, int ff, int width,
                 float limit, int relu_sq, hipStream_t s);
int mx_moe_topk(int* idx, float* wts, const float* z, const float* corr, long rows, int experts, int top,
                int groups, int keep, hipStream_t s);
}

namespace {

using at::Tensor;
using OptT = c10::optional<Tensor>;

hipStream_t stream() { return c10::hip::getCurrentHIPStream().stream(); }

bool is_act(const Tensor& t) { return t.scalar_type() == at::kFloat || t.scalar_type() == at::kBFloat16; }
int bf(const Tensor& t) { return t.scalar_type() == at::kBFloat16 ? 1 : 0; }

void chk(int rc, const char* what) { TORCH_CHECK(rc == 0, what, " failed (", rc, ")"); }

const float* opt_f32(const c10::optional<at::Tensor>& t, int64_t n, const char* what);

void check_f32(const Tensor& t, const char* n) {
  TORCH_CHECK(t.is_cuda() && t.scalar_type() == at::kFloat && t.is_contiguous(), n, ": fp32 contiguous GPU tensor");
}
void check_i32(const Tensor& t, const char* n) {
  TORCH_CHECK(t.is_cuda() && t.scalar_type() == at::kInt && t.is_contiguous(), n, ": int32 contiguous GPU tensor");
}
// 2-D rows with unit inner stride (views of a wider product are fine)
void check_rows(const Tensor& t, const char* n) {
  TORCH_CHECK(t.is_cuda() && is_act(t) && t.dim() == 2 && (t.size(1) == 1 || t.stride(1) == 1), n,
              ": 2-D fp32/bf16 GPU rows with unit inner stride");
}

// segment arrays: start [S+1], pos0 / slot / kv_len [>= S]
void check_segs(const Tensor& start, const Tensor& a, const Tensor& b, int64_t num) {
  check_i32(start, "seg.start");
  check_i32(a, "seg array");
  check_i32(b, "seg array");
  TORCH_CHECK(num >= 0 && start.numel() >= num + 1 && a.numel() >= num && b.numel() >= num, "segment arrays too short");
}

void embed_rows(Tensor out, Tensor ids, Tensor table, double scale, OptT positions, OptT freqs) {
  check_f32(out, "out");
  check_i32(ids, "ids");
  TORCH_CHECK(table.is_cuda() && is_act(table) && table.is_contiguous() && table.dim() == 2, "table");
  TORCH_CHECK(out.dim() == 2 && out.size(0) == ids.numel() && out.size(1) == table.size(1), "out shape");
  const int* pp = nullptr;
  const float* fp = nullptr;
  if (freqs) {
    TORCH_CHECK(positions, "positions go with the sinusoid frequencies");
    check_i32(*positions, "positions");
    check_f32(*freqs, "sinusoid frequencies");
    TORCH_CHECK(positions->numel() >= ids.numel() && freqs->numel() * 2 >= table.size(1), "positions / frequencies size");
    pp = positions->data_ptr<int>();
    fp = freqs->data_ptr<float>();
  }
  chk(mx_embed_rows(out.data_ptr<float>(), ids.data_ptr<int>(), table.data_ptr(), bf(table), (int)ids.numel(),
                    (int)table.size(1), (int)table.size(0), (float)scale, pp, fp, stream()), "embed_rows");
}

// x (fp32 residual) with y: x += ln(y), cast = x; without y: out = ln(x), or, without out, x = ln(x), cast = x
void layer_norm(Tensor x, OptT y, Tensor w, Tensor b, OptT out, OptT cast, double eps) {
  check_f32(x, "residual");
  TORCH_CHECK(x.dim() == 2, "residual 2-D");
  const int64_t rows = x.size(0), width = x.size(1);
  check_f32(w, "norm weight");
  check_f32(b, "norm bias");
  TORCH_CHECK(w.numel() == width && b.numel() == width, "norm weight / bias size");
  TORCH_CHECK(!(y && out), "out goes without y");
  const void* yp = nullptr;
  int ybf = 0;
  long ys = 0;
  if (y) {
    check_rows(*y, "y");
    TORCH_CHECK(y->size(0) == rows && y->size(1) == width, "y shape");
    yp = y->data_ptr();
    ybf = bf(*y);
    ys = y->stride(0);
  }
  int obf = 0;
  void *op = nullptr, *cp = nullptr;
  for (const OptT* t : {&out, &cast}) {
    if (!*t) continue;
    TORCH_CHECK((*t)->is_cuda() && (*t)->is_contiguous() && is_act(**t) && (*t)->sizes() == x.sizes(), "out / cast");
    obf = bf(**t);
  }
  if (out) op = out->data_ptr();
  if (cast) cp = cast->data_ptr();
  chk(mx_layer_norm(x.data_ptr<float>(), yp, ybf, ys, w.data_ptr<float>(), b.data_ptr<float>(), op, cp, obf,
                    (int)rows, (int)width, (float)eps, stream()), "layer_norm");
}

void tanh_cap(Tensor x, double cap) {
  check_f32(x, "x");
  TORCH_CHECK(cap > 0, "cap > 0");
  chk(mx_tanh_cap(x.data_ptr<float>(), x.numel(), (float)cap, stream()), "tanh_cap");
}

void add_rms_norm(Tensor x, OptT y, OptT wb, OptT add_vec, OptT next_w, OptT out, OptT cast, double eps) {
  check_f32(x, "residual");
  TORCH_CHECK(x.dim() == 2, "residual 2-D");
  const int64_t rows = x.size(0), width = x.size(1);
  const void* yp = nullptr;
  int ybf = 0;
  long ys = 0;
  if (y) {
    check_rows(*y, "y");
    TORCH_CHECK(y->size(0) == rows && y->size(1) == width && wb, "y shape / wb");
    check_f32(*wb, "wb");
    TORCH_CHECK(wb->numel() == width, "wb size");
    yp = y->data_ptr();
    ybf = bf(*y);
    ys = y->stride(0);
  }
  if (add_vec) { check_f32(*add_vec, "add_vec"); TORCH_CHECK(add_vec->numel() == width, "add_vec size"); }
  TORCH_CHECK((bool)next_w == (bool)out, "next_w and out go together");
  int obf = 0;
  if (out) {
    check_f32(*next_w, "next_w");
    TORCH_CHECK(next_w->numel() == width && out->is_cuda() && is_act(*out) && out->is_contiguous() &&
                out->numel() == rows * width, "out");
    obf = bf(*out);
  }
  if (cast) {
    TORCH_CHECK(cast->is_cuda() && is_act(*cast) && cast->is_contiguous() && cast->numel() == rows * width, "cast");
    TORCH_CHECK(!out || bf(*cast) == obf, "out and cast share a dtype");
    obf = bf(*cast);
  }
  chk(mx_add_rms_norm(x.data_ptr<float>(), yp, ybf, ys, wb ? wb->data_ptr<float>() : nullptr,
                      add_vec ? add_vec->data_ptr<float>() : nullptr, next_w ? next_w->data_ptr<float>() : nullptr,
                      out ? out->data_ptr() : nullptr, cast ? cast->data_ptr() : nullptr, obf, (int)rows,
                      (int)width, (float)eps, stream()), "add_rms_norm");
}

void head_rms_gate(Tensor out, Tensor o, Tensor w, Tensor gate, double eps, int64_t heads, int64_t dv, bool silu) {
  check_f32(o, "o");
  check_f32(w, "w");
  check_rows(gate, "gate");
  TORCH_CHECK(o.dim() == 2 && o.size(1) == heads * dv && w.numel() == dv && gate.size(0) == o.size(0) &&
              gate.size(1) == heads * dv, "head_rms_gate shapes");
  TORCH_CHECK(out.is_cuda() && is_act(out) && out.is_contiguous() && out.sizes() == o.sizes() &&
              bf(out) == bf(gate), "out");
  chk(mx_head_rms_gate(out.data_ptr(), bf(out), o.data_ptr<float>(), w.data_ptr<float>(), gate.data_ptr(),
                       bf(gate), gate.stride(0), o.size(0), (int)heads, (int)dv, (float)eps, silu ? 1 : 0,
                       stream()),
      "head_rms_gate");
}

void relu_sq(Tensor x) {
  TORCH_CHECK(x.is_cuda() && is_act(x) && x.is_contiguous(), "x");
  chk(mx_relu_sq(x.data_ptr(), bf(x), x.numel(), stream()), "relu_sq");
}

void relu_sq_rows(Tensor out, Tensor u) {
  check_rows(u, "u");
  TORCH_CHECK(out.is_cuda() && out.is_contiguous() && out.scalar_type() == u.scalar_type() && out.dim() == 2 &&
              out.size(0) == u.size(0) && out.size(1) >= 1 && out.size(1) <= u.size(1), "out");
  chk(mx_relu_sq_rows(out.data_ptr(), u.data_ptr(), bf(u), u.stride(0), u.size(0), (int)out.size(1), stream()),
      "relu_sq_rows");
}

void gather_add_rows(Tensor out, Tensor y, Tensor idx, Tensor w) {
  check_f32(out, "out");
  check_i32(idx, "idx");
  check_f32(w, "weights");
  TORCH_CHECK(y.is_cuda() && y.is_contiguous() && is_act(y) && y.dim() == 2 && out.dim() == 2 &&
              y.size(1) == out.size(1) && idx.dim() == 2 && idx.size(0) == out.size(0) && w.sizes() == idx.sizes(),
              "gather_add_rows shapes");
  chk(mx_gather_add_rows(out.data_ptr<float>(), y.data_ptr(), bf(y), idx.data_ptr<int>(), w.data_ptr<float>(),
                         out.size(0), (int)idx.size(1), (int)out.size(1), y.size(0), stream()), "gather_add_rows");
}

// out [M, N] = rows of a [M, K] (sorted by group, group g ends at offs[g]) times w[g]^T, w [G, N, K]; bf16
void grouped_gemm(Tensor out, Tensor a, Tensor w, Tensor offs) {
  check_i32(offs, "offsets");
  TORCH_CHECK(a.is_cuda() && a.is_contiguous() && a.scalar_type() == at::kBFloat16 && a.dim() == 2, "a: bf16 [M, K]");
  TORCH_CHECK(w.is_cuda() && w.is_contiguous() && w.scalar_type() == at::kBFloat16 && w.dim() == 3 &&
              w.size(2) == a.size(1) && offs.numel() == w.size(0), "w: bf16 [G, N, K], offsets [G]");
  TORCH_CHECK(out.is_cuda() && out.is_contiguous() && out.scalar_type() == at::kBFloat16 && out.dim() == 2 &&
              out.size(0) == a.size(0) && out.size(1) == w.size(1), "out: bf16 [M, N]");
  TORCH_CHECK(a.size(1) % 8 == 0 && a.size(1) >= 8, "K must be a multiple of 8");
  chk(mx_grouped_gemm(out.data_ptr(), a.data_ptr(), w.data_ptr(), offs.data_ptr<int>(), (int)w.size(0), a.size(0),
                      (int)w.size(1), (int)a.size(1), stream()), "grouped_gemm");
}

void clamp_swiglu(Tensor out, Tensor gu, double limit) {
  check_rows(gu, "gu");
  const int64_t ff = gu.size(1) / 2;
  TORCH_CHECK(out.is_cuda() && out.is_contiguous() && out.scalar_type() == gu.scalar_type() && out.dim() == 2 &&
              out.size(0) == gu.size(0) && out.size(1) == ff && ff >= 1, "out");
  chk(mx_clamp_swiglu(out.data_ptr(), gu.data_ptr(), bf(gu), gu.stride(0), gu.size(0), (int)ff, (float)limit,
                      stream()), "clamp_swiglu");
}

void side_gate(Tensor out, Tensor gpre, Tensor table, Tensor ids, int64_t col0) {
  check_i32(ids, "ids");
  TORCH_CHECK(gpre.is_cuda() && is_act(gpre) && gpre.is_contiguous() && gpre.dim() == 2, "gpre");
  TORCH_CHECK(out.is_cuda() && out.is_contiguous() && out.scalar_type() == gpre.scalar_type() &&
              out.sizes() == gpre.sizes(), "out");
  TORCH_CHECK(table.is_cuda() && table.is_contiguous() && table.dim() == 2 &&
              table.scalar_type() == gpre.scalar_type() && col0 >= 0 && col0 + gpre.size(1) <= table.size(1) &&
              ids.numel() == gpre.size(0), "table / ids");
  chk(mx_side_gate(out.data_ptr(), gpre.data_ptr(), table.data_ptr(), bf(gpre), table.size(1),
                   ids.data_ptr<int>(), (int)col0, gpre.size(0), (int)gpre.size(1), (int)table.size(0), stream()),
      "side_gate");
}

void scale_add_rows(Tensor out, Tensor y, OptT rows, Tensor weights, bool sigmoid) {
  check_f32(out, "out");
  TORCH_CHECK(y.is_cuda() && is_act(y) && y.is_contiguous() && y.dim() == 2 && out.dim() == 2 &&
              y.size(1) == out.size(1), "y");
  TORCH_CHECK(weights.is_cuda() && is_act(weights) && weights.is_contiguous() && weights.numel() == y.size(0),
              "weights");
  if (rows) { check_i32(*rows, "rows"); TORCH_CHECK(rows->numel() == y.size(0), "rows size"); }
  else TORCH_CHECK(y.size(0) == out.size(0), "identity rows need equal row counts");
  chk(mx_scale_add_rows(out.data_ptr<float>(), y.data_ptr(), bf(y), rows ? rows->data_ptr<int>() : nullptr,
                        weights.data_ptr(), bf(weights), sigmoid ? 1 : 0, y.size(0), (int)y.size(1),
                        (int)out.size(0), stream()), "scale_add_rows");
}

void short_conv_silu(Tensor out, Tensor x, Tensor w, OptT bias, Tensor hist, Tensor start, Tensor pos0, Tensor slot,
                     int64_t num_segs, int64_t max_rows) {
  check_rows(x, "x");
  TORCH_CHECK(out.is_cuda() && out.is_contiguous() && out.scalar_type() == x.scalar_type() &&
              out.sizes() == x.sizes(), "out");
  check_f32(w, "conv_w");
  if (bias) { check_f32(*bias, "conv bias"); TORCH_CHECK(bias->numel() == x.size(1), "conv bias size"); }
  check_f32(hist, "conv_state");
  const int64_t c = x.size(1), taps = w.size(1);
  TORCH_CHECK(w.dim() == 2 && w.size(0) == c && hist.dim() == 3 && hist.size(1) == taps - 1 && hist.size(2) == c,
              "conv shapes");
  check_segs(start, pos0, slot, num_segs);
  TORCH_CHECK(max_rows <= x.size(0), "max_rows");
  chk(mx_short_conv_silu(out.data_ptr(), x.data_ptr(), bf(x), x.stride(0), w.data_ptr<float>(),
                         bias ? bias->data_ptr<float>() : nullptr, hist.data_ptr<float>(),
                         start.data_ptr<int>(), pos0.data_ptr<int>(), slot.data_ptr<int>(), (int)num_segs,
                         (int)max_rows, (int)c, (int)taps, (int)hist.size(0), stream()), "short_conv_silu");
}

void gated_delta_rule(Tensor o, Tensor qkv, Tensor a, Tensor b, Tensor a_log, Tensor dt_bias, Tensor state,
                      Tensor start, Tensor pos0, Tensor slot, int64_t num_segs, int64_t heads, int64_t kv_heads,
                      int64_t dk, int64_t dv) {
  check_f32(o, "o");
  check_rows(qkv, "qkv");
  check_rows(a, "a");
  check_rows(b, "b");
  check_f32(a_log, "a_log");
  check_f32(dt_bias, "dt_bias");
  check_f32(state, "state");
  const int64_t t = qkv.size(0);
  TORCH_CHECK(heads >= 1 && kv_heads >= 1 && heads % kv_heads == 0 && dk >= 1 && dk <= mx_delta_max_dk() && dv >= 1,
              "delta rule sizes");
  TORCH_CHECK(qkv.size(1) == 2 * kv_heads * dk + heads * dv && a.size(0) == t && a.size(1) == heads * dk &&
              b.size(0) == t && b.size(1) == heads && a_log.numel() == heads && dt_bias.numel() == heads * dk &&
              o.numel() == t * heads * dv && a.scalar_type() == qkv.scalar_type() &&
              b.scalar_type() == qkv.scalar_type(), "delta rule shapes");
  TORCH_CHECK(state.dim() == 4 && state.size(1) == heads && state.size(2) == dk && state.size(3) == dv, "state");
  check_segs(start, pos0, slot, num_segs);
  auto f32 = qkv.options().dtype(at::kFloat);
  Tensor qn = at::empty({t, kv_heads, dk}, f32), kn = at::empty({t, kv_heads, dk}, f32);
  Tensor g = at::empty({t, heads, dk}, f32), beta = at::empty({t, heads}, f32);
  chk(mx_delta_prep(qn.data_ptr<float>(), kn.data_ptr<float>(), g.data_ptr<float>(), beta.data_ptr<float>(),
                    qkv.data_ptr(), bf(qkv), qkv.stride(0), a.data_ptr(), a.stride(0), b.data_ptr(), b.stride(0),
                    a_log.data_ptr<float>(), dt_bias.data_ptr<float>(), t, (int)heads, (int)kv_heads, (int)dk,
                    stream()), "delta_prep");
  chk(mx_delta_rule(o.data_ptr<float>(), qn.data_ptr<float>(), kn.data_ptr<float>(), g.data_ptr<float>(),
                    beta.data_ptr<float>(), qkv.data_ptr(), bf(qkv), qkv.stride(0), state.data_ptr<float>(),
                    start.data_ptr<int>(), pos0.data_ptr<int>(), slot.data_ptr<int>(), (int)num_segs, (int)heads,
                    (int)kv_heads, (int)dk, (int)dv, (int)state.size(0), stream()), "delta_rule");
}

void gated_linear_attention(Tensor o, Tensor qkv, Tensor a, Tensor a_bias, double tau, Tensor state, Tensor start,
                            Tensor pos0, Tensor slot, int64_t num_segs, int64_t max_rows, int64_t heads, int64_t dk,
                            int64_t dv) {
  check_f32(o, "o");
  check_rows(qkv, "qkv");
  check_rows(a, "a");
  check_f32(a_bias, "a_bias");
  check_f32(state, "state");
  const int64_t t = qkv.size(0);
  TORCH_CHECK(heads >= 1 && dk >= 1 && dk <= mx_gla_max_dk() && dv >= 1 && tau > 0, "linear attention sizes");
  TORCH_CHECK(qkv.size(1) >= heads * (2 * dk + dv) && a.size(0) == t && a.size(1) == heads * dk &&
              a_bias.numel() == heads * dk && o.numel() == t * heads * dv && a.scalar_type() == qkv.scalar_type(),
              "linear attention shapes");
  TORCH_CHECK(state.dim() == 4 && state.size(1) == heads && state.size(2) == dk && state.size(3) == dv, "state");
  check_segs(start, pos0, slot, num_segs);
  TORCH_CHECK(start.numel() >= num_segs + 1, "segments");
  chk(mx_gla_scan(o.data_ptr<float>(), qkv.data_ptr(), bf(qkv), qkv.stride(0), a.data_ptr(), a.stride(0),
                  a_bias.data_ptr<float>(), (float)tau, state.data_ptr<float>(), start.data_ptr<int>(),
                  pos0.data_ptr<int>(), slot.data_ptr<int>(), (int)num_segs, (int)std::max<int64_t>(max_rows, 0),
                  (int)heads, (int)dk, (int)dv, (int)state.size(0), stream()), "linear attention");
}

void pair_embed_add(Tensor x, Tensor ids, Tensor table, int64_t mul_prev, int64_t mul_cur, int64_t buckets,
                    Tensor start, Tensor pos0, Tensor slot, int64_t num_segs, Tensor last_tok, OptT embed,
                    double scale) {
  check_f32(x, "residual");
  if (embed)
    TORCH_CHECK(embed->is_cuda() && embed->is_contiguous() && embed->dim() == 2 && embed->size(1) == x.size(1) &&
                embed->scalar_type() == table.scalar_type(), "embedding table");
  check_i32(ids, "ids");
  check_i32(last_tok, "last tokens");
  TORCH_CHECK(table.is_cuda() && is_act(table) && table.is_contiguous() && table.dim() == 2, "table");
  TORCH_CHECK(x.dim() == 2 && x.size(0) == ids.numel() && x.size(1) == table.size(1) && buckets >= 1 &&
              table.size(0) == buckets + 1 && mul_prev >= 0 && mul_cur >= 0, "pair_embed_add shapes");
  check_segs(start, pos0, slot, num_segs);
  chk(mx_pair_embed_add(x.data_ptr<float>(), ids.data_ptr<int>(), table.data_ptr(), bf(table), (int)ids.numel(),
                        (int)table.size(1), (long)mul_prev, (long)mul_cur, (int)buckets, start.data_ptr<int>(),
                        pos0.data_ptr<int>(), slot.data_ptr<int>(), (int)num_segs, last_tok.data_ptr<int>(),
                        (int)last_tok.numel(), embed ? embed->data_ptr() : nullptr, embed ? (int)embed->size(0) : 0,
                        (float)scale, stream()), "pair_embed_add");
}

void add_scaled_rms_norm(Tensor x, OptT y1, OptT y2, double mult, OptT next_w, OptT out, double eps) {
  check_f32(x, "residual");
  TORCH_CHECK(x.dim() == 2, "residual 2-D");
  const int64_t rows = x.size(0), width = x.size(1);
  TORCH_CHECK((bool)next_w == (bool)out && (y1 || (!y2 && out)), "add_scaled_rms_norm arguments");
  const void *p1 = nullptr, *p2 = nullptr;
  int b1 = 0, b2 = 0;
  long s1 = 0, s2 = 0;
  if (y1) {
    check_rows(*y1, "y1");
    TORCH_CHECK(y1->size(0) == rows && y1->size(1) == width, "y1 shape");
    p1 = y1->data_ptr(); b1 = bf(*y1); s1 = y1->stride(0);
  }
  if (y2) {
    check_rows(*y2, "y2");
    TORCH_CHECK(y2->size(0) == rows && y2->size(1) == width, "y2 shape");
    p2 = y2->data_ptr(); b2 = bf(*y2); s2 = y2->stride(0);
  }
  void* op = nullptr;
  int obf = 0;
  if (out) {
    TORCH_CHECK(out->is_cuda() && out->is_contiguous() && is_act(*out) && out->sizes() == x.sizes(), "out");
    op = out->data_ptr();
    obf = bf(*out);
  }
  chk(mx_add_scaled_rms_norm(x.data_ptr<float>(), p1, b1, s1, p2, b2, s2, (float)mult,
                             opt_f32(next_w, width, "next norm weight"), op, obf, (int)rows, (int)width, (float)eps,
                             stream()), "add_scaled_rms_norm");
}

void dual_rms_mean(Tensor out, Tensor a, Tensor b, Tensor wa, Tensor wb, double eps, double scale) {
  check_f32(out, "out");
  check_rows(a, "a");
  check_rows(b, "b");
  check_f32(wa, "wa");
  check_f32(wb, "wb");
  const int64_t rows = a.size(0), width = a.size(1);
  TORCH_CHECK(b.sizes() == a.sizes() && b.scalar_type() == a.scalar_type() && out.dim() == 2 && out.size(0) == rows &&
              out.size(1) == width && wa.numel() == width && wb.numel() == width, "dual_rms_mean shapes");
  chk(mx_dual_rms_mean(out.data_ptr<float>(), a.data_ptr(), a.stride(0), b.data_ptr(), b.stride(0), bf(a),
                       wa.data_ptr<float>(), wb.data_ptr<float>(), (int)rows, (int)width, (float)eps, (float)scale,
                       stream()), "dual_rms_mean");
}

void sigmoid_gate(Tensor out, Tensor o, Tensor g) {
  check_f32(o, "o");
  check_rows(g, "g");
  TORCH_CHECK(o.dim() == 2 && g.size(0) == o.size(0) && g.size(1) == o.size(1), "sigmoid_gate shapes");
  TORCH_CHECK(out.is_cuda() && is_act(out) && out.is_contiguous() && out.sizes() == o.sizes() && bf(out) == bf(g),
              "out");
  chk(mx_sigmoid_gate(out.data_ptr(), bf(out), o.data_ptr<float>(), g.data_ptr(), bf(g), g.stride(0), o.size(0),
                      (int)o.size(1), stream()), "sigmoid_gate");
}

void latent_kv_write(Tensor dkv, Tensor w, double eps, Tensor table, int64_t dims, Tensor positions,
                     Tensor slots, Tensor cache, int64_t rank) {
  check_rows(dkv, "dkv");
  check_f32(w, "norm_w");
  check_f32(table, "rope table");
  check_i32(positions, "positions");
  check_i32(slots, "slot_mapping");
  const int64_t t = dkv.size(0), dr = dkv.size(1) - rank;
  TORCH_CHECK(rank >= 1 && dr >= 0 && dims % 2 == 0 && dims <= dr && w.numel() == rank && table.dim() == 2 &&
              table.size(1) == dims && positions.numel() >= t && slots.numel() >= t, "latent_kv_write shapes");
  TORCH_CHECK(cache.is_cuda() && cache.is_contiguous() && cache.dim() == 3 && cache.size(2) == rank + dr &&
              cache.scalar_type() == dkv.scalar_type(), "cache");
  chk(mx_latent_kv_write(dkv.data_ptr(), bf(dkv), dkv.stride(0), w.data_ptr<float>(), (float)eps,
                         table.data_ptr<float>(), (int)table.size(0), (int)dims, positions.data_ptr<int>(),
                         slots.data_ptr<int>(), cache.data_ptr(), bf(cache), cache.size(0) * cache.size(1), t,
                         (int)rank, (int)dr, stream()), "latent_kv_write");
}

void latent_q_rope(Tensor qn, Tensor qr, Tensor q, Tensor table, int64_t dims, Tensor positions, int64_t heads,
                   int64_t dn, int64_t dr) {
  check_f32(qn, "qn");
  check_f32(qr, "qr");
  check_rows(q, "q");
  check_f32(table, "rope table");
  check_i32(positions, "positions");
  const int64_t t = q.size(0);
  TORCH_CHECK(q.size(1) == heads * (dn + dr) && qn.numel() == t * heads * dn && qr.numel() == t * heads * dr &&
              dims % 2 == 0 && dims <= dr && table.dim() == 2 && table.size(1) == dims && positions.numel() >= t,
              "latent_q_rope shapes");
  chk(mx_latent_q_rope(qn.data_ptr<float>(), qr.data_ptr<float>(), q.data_ptr(), bf(q), q.stride(0),
                       table.data_ptr<float>(), (int)table.size(0), (int)dims, positions.data_ptr<int>(), t,
                       (int)heads, (int)dn, (int)dr, stream()), "latent_q_rope");
}

void latent_attention(Tensor out, Tensor qa, Tensor qr, Tensor cache, Tensor start, Tensor pos0, Tensor kv_len,
                      Tensor bt, int64_t num_segs, int64_t max_rows, double scale, int64_t rank, int64_t skip_from,
                      int64_t max_kv) {
  check_f32(out, "out");
  check_f32(qa, "qa");
  check_f32(qr, "qr");
  TORCH_CHECK(qa.dim() == 3 && qr.dim() == 3 && qa.size(2) == rank && out.sizes() == qa.sizes(), "qa / out");
  const int64_t heads = qa.size(0), t = qa.size(1), dr = qr.size(2);
  TORCH_CHECK(qr.size(0) == t && qr.size(1) == heads && rank <= mx_latent_max_rank(), "qr");
  TORCH_CHECK(cache.is_cuda() && cache.is_contiguous() && cache.dim() == 3 && cache.size(2) == rank + dr &&
              is_act(cache), "cache");
  check_segs(start, pos0, kv_len, num_segs);
  check_i32(bt, "block tables");
  TORCH_CHECK(bt.dim() == 2 && bt.size(0) >= num_segs && max_rows <= t, "block tables / max_rows");
  if (mx_latent_split_ws((int)heads, (int)rank, (int)dr)) {
    // key slices: enough workgroups to fill the chip (at most 16), at least ~64 keys per slice when
    // the longest context is known (max_kv; 0 inside captured graphs), scratch <= 256 MiB
    int64_t rows = std::max<int64_t>(1, std::min<int64_t>(t, num_segs * std::max<int64_t>(1, std::min(max_rows, skip_from > 0 ? skip_from - 1 : max_rows))));
    int64_t splits = std::max<int64_t>(1, std::min<int64_t>(16, 256 / rows));
    if (max_kv > 0) splits = std::max<int64_t>(1, std::min(splits, (max_kv + 63) / 64));
    while (splits > 1 && t * splits * heads * rank * 4 > (256LL << 20)) splits /= 2;
    auto f32 = qa.options();
    Tensor ws_acc = at::empty({t, splits, heads, rank}, f32), ws_ml = at::empty({t, splits, heads, 2}, f32);
    chk(mx_latent_attention_split(out.data_ptr<float>(), ws_acc.data_ptr<float>(), ws_ml.data_ptr<float>(),
                                  qa.data_ptr<float>(), qr.data_ptr<float>(), cache.data_ptr(), bf(cache),
                                  start.data_ptr<int>(), pos0.data_ptr<int>(), kv_len.data_ptr<int>(),
                                  bt.data_ptr<int>(), (int)bt.size(1), (int)num_segs, (int)max_rows, (int)heads,
                                  t, (int)rank, (int)dr, (int)cache.size(1), (int)cache.size(0), (float)scale,
                                  (int)skip_from, (int)splits, stream()), "latent_attention_split");
    return;
  }
  chk(mx_latent_attention(out.data_ptr<float>(), qa.data_ptr<float>(), qr.data_ptr<float>(), cache.data_ptr(),
                          bf(cache), start.data_ptr<int>(), pos0.data_ptr<int>(), kv_len.data_ptr<int>(),
                          bt.data_ptr<int>(), (int)bt.size(1), (int)num_segs, (int)max_rows, (int)heads, t,
                          (int)rank, (int)dr, (int)cache.size(1), (int)cache.size(0), (float)scale, (int)skip_from,
                          stream()),
      "latent_attention");
}

void causal_softmax(Tensor P, Tensor S, int64_t rows_per_head, int64_t first_pos, double scale) {
  check_f32(S, "S");
  TORCH_CHECK(S.dim() == 2 && P.is_cuda() && is_act(P) && P.is_contiguous() && P.sizes() == S.sizes() &&
              rows_per_head >= 1 && S.size(0) % rows_per_head == 0 && first_pos >= 0, "causal_softmax shapes");
  chk(mx_causal_softmax(P.data_ptr(), bf(P), S.data_ptr<float>(), S.size(0), (int)rows_per_head, (int)first_pos,
                        (int)S.size(1), (float)scale, stream()), "causal_softmax");
}

void moe_topk(Tensor idx, Tensor wts, Tensor z, Tensor corr, int64_t top, int64_t groups, int64_t keep) {
  check_i32(idx, "idx");
  check_f32(wts, "wts");
  check_f32(z, "z");
  check_f32(corr, "correction");
  TORCH_CHECK(z.dim() == 2 && corr.numel() == z.size(1) && idx.numel() == z.size(0) * top &&
              wts.numel() == z.size(0) * top, "moe_topk shapes");
  chk(mx_moe_topk(idx.data_ptr<int>(), wts.data_ptr<float>(), z.data_ptr<float>(), corr.data_ptr<float>(),
                  z.size(0), (int)z.size(1), (int)top, (int)groups, (int)keep, stream()), "moe_topk");
}

void moe_top_logits(Tensor idx, Tensor wts, Tensor z, int64_t top) {
  check_i32(idx, "idx");
  check_f32(wts, "wts");
  check_f32(z, "z");
  TORCH_CHECK(z.dim() == 2 && top >= 1 && top <= z.size(1) && idx.numel() == z.size(0) * top &&
              wts.numel() == z.size(0) * top, "moe_top_logits shapes");
  chk(mx_moe_top_logits(idx.data_ptr<int>(), wts.data_ptr<float>(), z.data_ptr<float>(), z.size(0), (int)z.size(1),
                        (int)top, stream()), "moe_top_logits");
}

void moe_route_top_logits(Tensor idx, Tensor wts, Tensor h, Tensor router, OptT bias, int64_t top) {
  check_i32(idx, "idx");
  check_f32(wts, "wts");
  check_rows(h, "h");
  check_f32(router, "router");
  TORCH_CHECK(router.dim() == 2 && router.size(1) == h.size(1) && top >= 1 && top <= router.size(0) &&
              idx.numel() == h.size(0) * top && wts.numel() == h.size(0) * top, "moe_route_top_logits shapes");
  if (bias) {
    check_f32(*bias, "router bias");
    TORCH_CHECK(bias->numel() == router.size(0), "router bias size");
  }
  chk(mx_moe_route_top_logits(idx.data_ptr<int>(), wts.data_ptr<float>(), h.data_ptr(), bf(h), h.stride(0),
                              router.data_ptr<float>(), bias ? bias->data_ptr<float>() : nullptr, h.size(0),
                              (int)router.size(0), (int)router.size(1), (int)top, stream()), "moe_route_top_logits");
}

// relu_sq: the experts' first matrix is [ff, width] (up alone) instead of [2 ff, width] (gate | up)
void moe_pairs(Tensor out, Tensor h, Tensor idx, Tensor wts, Tensor wgu, Tensor wdown, double limit, bool relu_sq) {
  check_f32(out, "out");
  check_rows(h, "h");
  check_i32(idx, "idx");
  check_f32(wts, "wts");
  TORCH_CHECK(wgu.is_cuda() && wgu.is_contiguous() && wgu.dim() == 3 && wdown.is_cuda() && wdown.is_contiguous() &&
              wdown.dim() == 3 && wgu.scalar_type() == h.scalar_type() && wdown.scalar_type() == h.scalar_type(),
              "expert weights");
  const int64_t rows = h.size(0), width = h.size(1), experts = wgu.size(0);
  const int64_t ff = relu_sq ? wgu.size(1) : wgu.size(1) / 2;
  TORCH_CHECK(idx.dim() == 2 && idx.size(0) == rows && wts.sizes() == idx.sizes(), "idx / wts");
  const int64_t top = idx.size(1);
  TORCH_CHECK(wgu.size(2) == width && wdown.size(0) == experts && wdown.size(1) == width && wdown.size(2) == ff &&
              wgu.size(1) == (relu_sq ? ff : 2 * ff) && out.dim() == 2 && out.size(0) == rows && out.size(1) == width,
              "moe_pairs shapes");
  TORCH_CHECK(((uintptr_t)h.data_ptr()) % 16 == 0, "h alignment");
  Tensor y = at::empty({rows * top, ff}, h.options());
  chk(mx_moe_pairs(out.data_ptr<float>(), y.data_ptr(), h.data_ptr(), bf(h), h.stride(0), idx.data_ptr<int>(),
                   wts.data_ptr<float>(), wgu.data_ptr(), wdown.data_ptr(), rows, (int)top, (int)experts, (int)ff,
                   (int)width, (float)limit, relu_sq ? 1 : 0, stream()), "moe_pairs");
}

void gelu_glu(Tensor out, Tensor gu, bool relu) {
  check_rows(gu, "gu");
  const int64_t ff = gu.size(1) / 2;
  TORCH_CHECK(out.is_cuda() && out.is_contiguous() && out.scalar_type() == gu.scalar_type() && out.dim() == 2 &&
              out.size(0) == gu.size(0) && out.size(1) == ff && ff >= 1 && gu.size(1) == 2 * ff, "out");
  chk(mx_gelu_glu(out.data_ptr(), gu.data_ptr(), bf(gu), gu.stride(0), gu.size(0), (int)ff, relu ? 1 : 0, stream()),
      "gelu_glu");
}

const float* opt_f32(const OptT& t, int64_t n, const char* what) {
  if (!t) return nullptr;
  check_f32(*t, what);
  TORCH_CHECK(t->numel() == n, what, ": size");
  return t->data_ptr<float>();
}

// paged caches [blocks, block_size, row]
void check_cache(const Tensor& c, int64_t row, const char* n) {
  TORCH_CHECK(c.is_cuda() && c.is_contiguous() && c.dim() == 3 && c.size(2) == row && is_act(c) &&
              c.size(0) * c.size(1) < (1LL << 31), n, ": paged cache [blocks, block_size, ", row, "]");
}

void attn_prep(Tensor q, Tensor qkv, int64_t nq, int64_t nk, OptT wq, OptT wk, double eps, OptT table,
               int64_t rot_dims, int64_t head_dim, Tensor positions, Tensor slots, OptT k_cache_, OptT v_cache_) {
  check_f32(q, "q");
  check_rows(qkv, "qkv");
  check_i32(positions, "positions");
  check_i32(slots, "slot_mapping");
  const int64_t t = qkv.size(0), nv = qkv.size(1) - nq - nk;
  TORCH_CHECK(nq >= 1 && head_dim >= 1 && nq % head_dim == 0 && nk % head_dim == 0 &&
              rot_dims >= 0 && rot_dims % 2 == 0 && rot_dims <= head_dim && q.numel() == t * nq &&
              positions.numel() >= t && slots.numel() >= t, "attn_prep shapes");
  if (!k_cache_ || !v_cache_) {
    // queries alone (a layer that attends to another layer's keys and values)
    TORCH_CHECK(!k_cache_ && !v_cache_ && nk == 0 && nv == 0 && !wk, "attn_prep: no caches goes with rows of q alone");
    const float* tq = nullptr;
    int64_t tr = 0;
    if (table && rot_dims > 0) {
      check_f32(*table, "rope table");
      TORCH_CHECK(table->dim() == 2 && table->size(1) == rot_dims, "rope table shape");
      tq = table->data_ptr<float>();
      tr = table->size(0);
    }
    chk(mx_attn_prep(q.data_ptr<float>(), qkv.data_ptr(), bf(qkv), qkv.stride(0), (int)nq, 0, 0,
                     opt_f32(wq, nq, "q norm"), nullptr, (float)eps, tq, (int)tr, (int)rot_dims, (int)head_dim,
                     positions.data_ptr<int>(), slots.data_ptr<int>(), nullptr, nullptr, bf(qkv), 0, t, stream()),
        "attn_prep");
    return;
  }
  const Tensor& k_cache = *k_cache_;
  const Tensor& v_cache = *v_cache_;
  TORCH_CHECK(nk >= 1 && nv >= 1, "attn_prep shapes");
  check_cache(k_cache, nk, "k_cache");
  check_cache(v_cache, nv, "v_cache");
  TORCH_CHECK(k_cache.scalar_type() == v_cache.scalar_type() && k_cache.size(0) == v_cache.size(0) &&
              k_cache.size(1) == v_cache.size(1), "k / v caches differ");
  const float* tp = nullptr;
  int64_t trows = 0;
  if (table && rot_dims > 0) {
    check_f32(*table, "rope table");
    TORCH_CHECK(table->dim() == 2 && table->size(1) == rot_dims, "rope table shape");
    tp = table->data_ptr<float>();
    trows = table->size(0);
  }
  chk(mx_attn_prep(q.data_ptr<float>(), qkv.data_ptr(), bf(qkv), qkv.stride(0), (int)nq, (int)nk, (int)nv,
                   opt_f32(wq, nq, "q norm"), opt_f32(wk, nk, "k norm"), (float)eps, tp, (int)trows, (int)rot_dims,
                   (int)head_dim, positions.data_ptr<int>(), slots.data_ptr<int>(), k_cache.data_ptr(),
                   v_cache.data_ptr(), bf(k_cache), k_cache.size(0) * k_cache.size(1), t, stream()), "attn_prep");
}

void conv_attn_prep(Tensor q, Tensor qkv, int64_t nq, int64_t nk, Tensor conv_w, Tensor hist, Tensor start,
                    Tensor pos0, Tensor slot, int64_t num_segs, OptT wq, OptT wk, double eps, int64_t head_dim,
                    Tensor slots, Tensor k_cache, Tensor v_cache) {
  check_f32(q, "q");
  check_rows(qkv, "qkv");
  check_i32(slots, "slot_mapping");
  check_f32(conv_w, "conv_w");
  check_f32(hist, "conv_state");
  const int64_t t = qkv.size(0), c = qkv.size(1), nv = c - nq - nk;
  TORCH_CHECK(nq >= 1 && nk >= 1 && nv >= 1 && head_dim >= 1 && nq % head_dim == 0 && nk % head_dim == 0 &&
              q.numel() == t * nq && slots.numel() >= t, "conv_attn_prep shapes");
  const int64_t taps = conv_w.dim() == 2 ? conv_w.size(1) : 0;
  TORCH_CHECK(conv_w.dim() == 2 && conv_w.size(0) == c && taps >= 1 && taps <= 16 && hist.dim() == 3 &&
              hist.size(1) == taps - 1 && hist.size(2) == c, "conv shapes");
  check_segs(start, pos0, slot, num_segs);
  check_cache(k_cache, nk, "k_cache");
  check_cache(v_cache, nv, "v_cache");
  TORCH_CHECK(k_cache.scalar_type() == v_cache.scalar_type() && k_cache.size(0) == v_cache.size(0) &&
              k_cache.size(1) == v_cache.size(1), "k / v caches differ");
  chk(mx_conv_attn_prep(q.data_ptr<float>(), qkv.data_ptr(), bf(qkv), qkv.stride(0), (int)nq, (int)nk, (int)nv,
                        conv_w.data_ptr<float>(), (int)taps, hist.data_ptr<float>(), start.data_ptr<int>(),
                        pos0.data_ptr<int>(), slot.data_ptr<int>(), (int)num_segs, (int)hist.size(0),
                        opt_f32(wq, head_dim, "q norm"), opt_f32(wk, head_dim, "k norm"), (float)eps, (int)head_dim,
                        slots.data_ptr<int>(), k_cache.data_ptr(), v_cache.data_ptr(), bf(k_cache),
                        k_cache.size(0) * k_cache.size(1), t, stream()), "conv_attn_prep");
}

void window_attention(Tensor out, Tensor q, Tensor k_cache, Tensor v_cache, Tensor start, Tensor pos0, Tensor kv_len,
                      Tensor bt, int64_t num_segs, int64_t max_rows, int64_t heads, int64_t maps, int64_t kv_heads,
                      int64_t dk, int64_t dv, int64_t window, double scale, bool sigmoid, OptT r1, OptT r2, OptT pb,
                      int64_t skip_from, double softcap, c10::optional<double> sink, bool blocks,
                      int64_t keep_first, OptT dist_bias) {
  check_f32(out, "out");
  check_f32(q, "q");
  TORCH_CHECK(keep_first >= 0 && (!blocks || window >= 1), "window attention mask");
  if (dist_bias) {
    check_f32(*dist_bias, "distance bias");
    TORCH_CHECK(dist_bias->dim() == 2 && dist_bias->size(0) >= 1 && dist_bias->size(1) == heads * maps,
                "distance bias [distances, heads]");
  }
  TORCH_CHECK(heads >= 1 && maps >= 1 && kv_heads >= 1 && heads % kv_heads == 0 && dk >= 1 && dv >= 1 &&
              dv <= mx_window_max_dv(), "window attention sizes");
  const int64_t hq = heads * maps, t = q.size(0);
  TORCH_CHECK(q.dim() == 2 && q.size(1) == hq * dk && out.numel() == t * hq * dv, "q / out");
  check_cache(k_cache, kv_heads * maps * dk, "k_cache");
  check_cache(v_cache, kv_heads * dv, "v_cache");
  TORCH_CHECK(k_cache.scalar_type() == v_cache.scalar_type() && k_cache.size(0) == v_cache.size(0) &&
              k_cache.size(1) == v_cache.size(1), "k / v caches differ");
  check_segs(start, pos0, kv_len, num_segs);
  check_i32(bt, "block tables");
  TORCH_CHECK(bt.dim() == 2 && bt.size(0) >= num_segs && max_rows <= t, "block tables / max_rows");
  TORCH_CHECK((bool)r1 == (bool)r2, "r1 and r2 go together");
  chk(mx_window_attention(out.data_ptr<float>(), q.data_ptr<float>(), k_cache.data_ptr(), v_cache.data_ptr(),
                          bf(k_cache), start.data_ptr<int>(), pos0.data_ptr<int>(), kv_len.data_ptr<int>(),
                          bt.data_ptr<int>(), (int)bt.size(1), (int)num_segs, t, (int)heads, (int)maps, (int)kv_heads,
                          (int)dk, (int)dv, (int)window, (float)scale, sigmoid ? 1 : 0, opt_f32(r1, hq, "r1"),
                          opt_f32(r2, hq, "r2"), opt_f32(pb, hq, "pb"), (int)k_cache.size(1), (int)k_cache.size(0),
                          (int)skip_from, (float)softcap, sink ? 1 : 0, sink ? (float)*sink : 0.f, blocks ? 1 : 0,
                          (int)keep_first, dist_bias ? dist_bias->data_ptr<float>() : nullptr,
                          dist_bias ? (int)dist_bias->size(0) : 0, stream()),
      "window_attention");
}

void band_weights(Tensor S, int64_t rows, int64_t first_pos, int64_t key0, int64_t heads, int64_t maps,
                  int64_t kv_heads, int64_t window, double scale, bool sigmoid, OptT r1, OptT r2, OptT pb,
                  double softcap, c10::optional<double> sink, bool blocks, int64_t keep_first, int64_t ext,
                  OptT dist_bias) {
  check_f32(S, "S");
  TORCH_CHECK(keep_first >= 0 && ext >= 0 && ext <= key0 && ext <= S.size(2) && (!blocks || window >= 1),
              "band_weights mask");
  if (dist_bias) {
    check_f32(*dist_bias, "distance bias");
    TORCH_CHECK(dist_bias->dim() == 2 && dist_bias->size(0) >= 1 && dist_bias->size(1) == heads * maps,
                "distance bias [distances, heads]");
  }
  TORCH_CHECK(S.dim() == 3 && heads >= 1 && kv_heads >= 1 && heads % kv_heads == 0 && maps >= 1 &&
              S.size(0) == kv_heads * maps && rows >= 1 && S.size(1) == heads / kv_heads * rows && first_pos >= 0 &&
              key0 >= 0, "band_weights shapes");
  TORCH_CHECK((bool)r1 == (bool)r2, "r1 and r2 go together");
  const int64_t hq = heads * maps;
  chk(mx_band_weights(S.data_ptr<float>(), (int)S.size(0), (int)S.size(1), (int)rows, (int)S.size(2), (int)first_pos,
                      (int)key0, (int)heads, (int)maps, (int)kv_heads, (int)window, (float)scale, sigmoid ? 1 : 0,
                      opt_f32(r1, hq, "r1"), opt_f32(r2, hq, "r2"), opt_f32(pb, hq, "pb"), (float)softcap, sink ? 1 : 0,
                      sink ? (float)*sink : 0.f, blocks ? 1 : 0, (int)keep_first, (int)ext,
                      dist_bias ? dist_bias->data_ptr<float>() : nullptr, dist_bias ? (int)dist_bias->size(0) : 0,
                      stream()), "band_weights");
}

void diff_combine(Tensor out, Tensor a, Tensor gate, double lam, double post, double eps, int64_t heads, int64_t dv) {
  check_f32(a, "a");
  check_rows(gate, "gate");
  const int64_t t = gate.size(0);
  TORCH_CHECK(a.numel() == t * heads * 2 * dv && gate.size(1) == heads, "diff_combine shapes");
  TORCH_CHECK(out.is_cuda() && is_act(out) && out.is_contiguous() && out.numel() == t * heads * dv &&
              bf(out) == bf(gate), "out");
  chk(mx_diff_combine(out.data_ptr(), bf(out), a.data_ptr<float>(), gate.data_ptr(), bf(gate), gate.stride(0), t,
                      (int)heads, (int)dv, (float)lam, (float)post, (float)eps, stream()), "diff_combine");
}

void ssd_scan(Tensor y, Tensor xbc, Tensor dt, Tensor a_log, Tensor dt_bias, Tensor d_skip, Tensor state,
              Tensor start, Tensor pos0, Tensor slot, int64_t num_segs, int64_t heads, int64_t groups, int64_t n,
              int64_t dv) {
  check_f32(y, "y");
  check_rows(xbc, "xbc");
  check_rows(dt, "dt");
  check_f32(a_log, "a_log");
  check_f32(dt_bias, "dt_bias");
  check_f32(d_skip, "D");
  check_f32(state, "state");
  const int64_t t = xbc.size(0);
  TORCH_CHECK(heads >= 1 && groups >= 1 && heads % groups == 0 && n >= 1 && n <= mx_ssd_max_state() && dv >= 1,
              "state-space sizes");
  TORCH_CHECK(xbc.size(1) == heads * dv + 2 * groups * n && dt.size(0) == t && dt.size(1) == heads &&
              dt.scalar_type() == xbc.scalar_type() && a_log.numel() == heads && dt_bias.numel() == heads &&
              d_skip.numel() == heads && y.numel() == t * heads * dv, "state-space shapes");
  TORCH_CHECK(state.dim() == 4 && state.size(1) == heads && state.size(2) == n && state.size(3) == dv, "state");
  check_segs(start, pos0, slot, num_segs);
  chk(mx_ssd_scan(y.data_ptr<float>(), xbc.data_ptr(), bf(xbc), xbc.stride(0), dt.data_ptr(), dt.stride(0),
                  a_log.data_ptr<float>(), dt_bias.data_ptr<float>(), d_skip.data_ptr<float>(),
                  state.data_ptr<float>(), start.data_ptr<int>(), pos0.data_ptr<int>(), slot.data_ptr<int>(),
                  (int)num_segs, (int)heads, (int)groups, (int)n, (int)dv, (int)state.size(0), stream()), "ssd_scan");
}

void gate_group_norm(Tensor out, Tensor y, Tensor z, Tensor w, double eps, int64_t groups) {
  check_f32(y, "y");
  check_rows(z, "z");
  check_f32(w, "w");
  TORCH_CHECK(y.dim() == 2 && z.size(0) == y.size(0) && z.size(1) == y.size(1) && w.numel() == y.size(1) &&
              groups >= 1 && y.size(1) % groups == 0, "gate_group_norm shapes");
  TORCH_CHECK(out.is_cuda() && is_act(out) && out.is_contiguous() && out.sizes() == y.sizes() && bf(out) == bf(z),
              "out");
  chk(mx_gate_group_norm(out.data_ptr(), bf(out), y.data_ptr<float>(), z.data_ptr(), bf(z), z.stride(0),
                         w.data_ptr<float>(), y.size(0), (int)groups, (int)(y.size(1) / groups), (float)eps, stream()),
      "gate_group_norm");
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.def("embed_rows", &embed_rows);
  m.def("add_rms_norm", &add_rms_norm);
  m.def("layer_norm", &layer_norm);
  m.def("tanh_cap", &tanh_cap);
  m.def("conv_attn_prep", &conv_attn_prep);
  m.def("moe_top_logits", &moe_top_logits);
  m.def("moe_route_top_logits", &moe_route_top_logits);
  m.def("head_rms_gate", &head_rms_gate);
  m.def("relu_sq", &relu_sq);
  m.def("relu_sq_rows", &relu_sq_rows);
  m.def("gather_add_rows", &gather_add_rows);
  m.def("grouped_gemm", &grouped_gemm);
  m.def("clamp_swiglu", &clamp_swiglu);
  m.def("side_gate", &side_gate);
  m.def("scale_add_rows", &scale_add_rows);
  m.def("short_conv_silu", &short_conv_silu);
  m.def("gated_delta_rule", &gated_delta_rule);
  m.def("gated_linear_attention", &gated_linear_attention);
  m.def("pair_embed_add", &pair_embed_add);
  m.def("add_scaled_rms_norm", &add_scaled_rms_norm);
  m.def("dual_rms_mean", &dual_rms_mean);
  m.def("sigmoid_gate", &sigmoid_gate);
  m.def("latent_kv_write", &latent_kv_write);
  m.def("latent_q_rope", &latent_q_rope);
  m.def("latent_attention", &latent_attention);
  m.def("causal_softmax", &causal_softmax);
  m.def("moe_topk", &moe_topk);
  m.def("moe_pairs", &moe_pairs);
  m.def("gelu_glu", &gelu_glu);
  m.def("attn_prep", &attn_prep);
  m.def("window_attention", &window_attention);
  m.def("band_weights", &band_weights);
  m.def("diff_combine", &diff_combine);
  m.def("ssd_scan", &ssd_scan);
  m.def("gate_group_norm", &gate_group_norm);
  m.def("window_max_dv", []() { return (int64_t)mx_window_max_dv(); });
  m.def("ssd_max_state", []() { return (int64_t)mx_ssd_max_state(); });
  m.def("delta_max_dk", []() { return (int64_t)mx_delta_max_dk(); });
  m.def("latent_max_rank", []() { return (int64_t)mx_latent_max_rank(); });
}
