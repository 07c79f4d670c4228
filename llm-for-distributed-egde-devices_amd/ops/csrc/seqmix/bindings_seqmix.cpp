// Python bindings of the ragged-step kernels (seqmix.hip): shape / dtype / device checks, outputs
// from torch's caching allocator, launches on torch's current HIP stream.  Activations are fp32 or
// bf16 (one flag per call, taken from the tensors); metadata tensors are int32 on the device.
#include <torch/extension.h>
#include <c10/hip/HIPStream.h>
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <hip/hip_runtime.h>

#include <optional>

extern "C" {
int edge_sm_embed(const int64_t* ids, const void* table, float* out, int rows, int W, int V, float scale, int f32,
                  hipStream_t st);
int edge_sm_scalar_norm(const float* x, const float* gain, void* y, int rows, int W, float eps, int f32, hipStream_t st);
int edge_sm_relu2(const void* u, int ld, int c0, void* y, int rows, int C, int f32, hipStream_t st);
int edge_sm_cat_cast(const float* a, const float* b, void* y, int rows, int W, int f32, hipStream_t st);
int edge_sm_combine(float* x, const void* l, const void* r, const float* wl, const float* wr, const void* extra,
                    int rows, int W, float eps, int f32, hipStream_t st);
int edge_sm_gated_norm(const float* y, const void* z, int z_ld, const float* w, void* out, int rows, int C, int groups,
                       float eps, int f32, hipStream_t st);
int edge_sm_rope_write(const void* proj, int ld, const int* tok_seq, const int* tok_pos, const int* seq_slot,
                       const int* ptab, int ptab_ld, const float* cs, void* q_out, void* kp, void* vp, int rows,
                       int H, int G, int D, int Dv, int rot, int page, int f32, hipStream_t st);
int edge_sm_group_norm(const float* x, const float* w, void* y, int rows, int W, int groups, float eps, int f32,
                       hipStream_t st);
int edge_sm_group_norm_residual(float* x, const void* y, const void* parts, const float* pw, int K, const float* w,
                                int rows, int W, int groups, float eps, float mult, int f32, hipStream_t st);
int edge_sm_glu_silu(const void* u, int ld, void* y, const float* row_w, int rows, int ff, int f32, hipStream_t st);
int edge_sm_delta_prep_head(const void* qkv, int Cq, const void* u, int ld, int b0, int a0, const float* dt_bias,
                            const float* A_log, float* prep, int rows, int H, int G, int N, int f32, hipStream_t st);
int edge_sm_pool_blocks(const void* kp, const void* vp, float* kb, float* vb, const int* seq_slot,
                        const int* seq_start, const int* seq_len, const int* ptab, int ptab_ld, int n, int max_blocks,
                        int G, int D, int Dv, int page, int PB, int pool, int f32, hipStream_t st);
int edge_sm_attention(const void* q, const void* gate, int gate_ld, const void* kp, const void* vp, const float* kb,
                      const float* vb, const int* tok_seq, const int* tok_pos, const int* seq_slot, const int* ptab,
                      int ptab_ld, void* out, int rows, int H, int G, int D, int Dv, int page, int PB, float scale,
                      int window, int pool, int f32, int nsplit, float* part, int kld, int vld, int chunked, float cap,
                      const float* slopes, const float* sink, int gate_elem, int keep_first, hipStream_t st);
size_t edge_sm_attention_part_floats(int rows, int H, int G, int D, int Dv, int nsplit);
int edge_sm_attention_mfma(const void* q, const void* gate, int gate_ld, const void* kp, const void* vp,
                           const float* kb, const float* vb, const int* seq_slot, const int* seq_start,
                           const int* seq_len, const int* seq_off, const int* ptab, int ptab_ld, void* out, int n,
                           int qtiles, int H, int G, int D, int Dv, int page, int PB, float scale, int window,
                           int pool, int kld, int vld, int chunked, float cap, const float* slopes, const float* sink,
                           int gate_elem, int keep_first, hipStream_t st);
int edge_sm_conv_silu(const void* u, int ld, int c0, int C, const float* w, const float* bias, void* state,
                      const int* tok_seq, const int* tok_pos, const int* seq_slot, const int* seq_start,
                      const int* seq_len, const int* seq_off, void* out, int rows, int n, int taps, int f32,
                      int max_len, hipStream_t st);
int edge_sm_ssd_scan(const void* xbc, int Cx, const void* u, int ld, int dt0, const float* dt_bias, const float* A_log,
                     const float* Dp, float* state, const int* seq_slot, const int* seq_start, const int* seq_len,
                     const int* seq_off, float* y, int n, int Hs, int P, int N, int groups, int f32, hipStream_t st);
int edge_sm_ssd_chunked(const void* xbc, int Cx, const void* u, int ld, int dt0, const float* dt_bias,
                        const float* A_log, const float* Dp, float* state, const int* seq_slot, const int* seq_start,
                        const int* seq_len, const int* seq_off, float* y, float* sloc, float* cdec, int n,
                        int max_chunks, int Hs, int P, int N, int groups, int f32, hipStream_t st);
int edge_sm_embed_bigram(const int64_t* ids, const void* table, const void* bigram, int64_t* prev_tok, const int* tok_seq,
                         const int* tok_pos, const int* seq_slot, const int* seq_start, const int* seq_len,
                         const int* seq_off, float* out, int rows, int n, int W, int V, long buckets, long mul_prev,
                         long mul_cur, int f32, hipStream_t st);
int edge_sm_canon(const float* x, int W, const float* w, float* state, const int* tok_seq, const int* tok_pos,
                  const int* seq_slot, const int* seq_start, const int* seq_len, const int* seq_off, void* out, int rows,
                  int n, int taps, int max_len, int f32, hipStream_t st);
int edge_sm_layer_norm(const float* x, const float* w, const float* b, void* y, int rows, int W, float eps, int f32,
                       hipStream_t st);
int edge_sm_ln_residual(float* x, const void* y, const void* parts, const float* pw, int K, const float* w, const float* b,
                        int rows, int W, float eps, int f32, hipStream_t st);
int edge_sm_rms_cols(const void* u, int ld, int c0, int C, const float* w, void* y, int rows, float eps, int f32,
                     hipStream_t st);
int edge_sm_head_norm_gate(const float* y, const void* z, int z_ld, const float* w, void* out, int rows, int H, int P,
                           float eps, int silu, int f32, hipStream_t st);
int edge_sm_glu_clamp(const void* u, int ld, void* y, int rows, int ff, float limit, int f32, hipStream_t st);
int edge_sm_latent_write(const void* u, int ld, int c0, const float* w, float eps, const void* q, const void* q_lat,
                         long ql_t, long ql_h, const int* tok_seq, const int* tok_pos, const int* seq_slot, const int* ptab,
                         int ptab_ld, const float* cs, void* pages, void* qc, int rows, int H, int D, int R, int kvr, int rot,
                         int page, int f32, hipStream_t st);
int edge_sm_delta_prep(const void* qkv, int Cq, const void* u, int ld, int b0, const float* a, const float* dt_bias,
                       const float* A_log, float* prep, int rows, int H, int G, int N, int f32, hipStream_t st);
int edge_sm_delta_scan(const float* prep, int prep_ld, const void* qkv, int Cq, float* state, const int* seq_slot,
                       const int* seq_start, const int* seq_len, const int* seq_off, float* y, int n, int H, int G, int N,
                       int P, int GD, int f32, hipStream_t st);
int edge_sm_moe_route(const void* h, int W, const float* router, const float* bias, int E, int top, float scale, float* z,
                      int* idx, float* wts, int rows, int sigm, int f32, hipStream_t st);
int edge_sm_hyper_read_norm(const float* X, const float* in_w, const float* w, void* y, int rows, int S, int W, float eps,
                            int f32, hipStream_t st);
int edge_sm_hyper_update(float* X, const float* mix, const float* out_w, const void* y, const void* parts, const float* pw,
                         int K, int rows, int S, int W, const float* in2, const float* w2, void* h, float eps, int f32,
                         hipStream_t st);
int edge_sm_poly_norm(const void* z, int ld, const float* coef, void* y, int rows, int F, float eps, int f32,
                      hipStream_t st);
int edge_sm_qk_norm_rope_write(const void* proj, int ld, const int* tok_seq, const int* tok_pos, const int* seq_slot,
                               const int* ptab, int ptab_ld, const float* qw, const float* kw, float eps, const float* cs,
                               const float* vcs, const float* temp, void* q_out, void* kp, void* vp, int rows, int H, int G,
                               int D, int Dv, int rot, int page, int f32, hipStream_t st);
int edge_sm_unrotate_gate(const void* a, const void* gate, int gate_ld, const int* tok_pos, const float* vcs, void* out,
                          int rows, int HD, int Dv, int f32, hipStream_t st);
int edge_sm_moe_experts(const void* h, int W, const int* idx, int top, const void* w_gu, const void* w_down, int ff,
                        float limit, int silu, const float* in_w, void* y, void* out, int rows, int E, int f32,
                        hipStream_t st);
}

namespace {

hipStream_t stream() { return c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream(); }

void check(int rc, const char* what) {
  TORCH_CHECK(rc == 0, what, ": launch failed (", rc, rc > 0 ? std::string(": ") + hipGetErrorString((hipError_t)rc) : "",
              ")");
}

bool is_act(const at::Tensor& t) { return t.scalar_type() == at::kFloat || t.scalar_type() == at::kBFloat16; }
int f32(const at::Tensor& t) { return t.scalar_type() == at::kFloat ? 1 : 0; }
at::ScalarType act_type(bool f) { return f ? at::kFloat : at::kBFloat16; }

// a [rows, cols] view whose rows are contiguous (stride(1) == 1): returns the row stride
int row_ld(const at::Tensor& t, const char* name) {
  TORCH_CHECK(t.is_cuda() && t.dim() == 2 && (t.size(1) == 0 || t.stride(1) == 1), name, ": rows must be contiguous");
  return (int)t.stride(0);
}
void chk_i32(const at::Tensor& t, const char* name) {
  TORCH_CHECK(t.is_cuda() && t.scalar_type() == at::kInt && t.is_contiguous(), name, ": int32 device tensor expected");
}
void chk_f32(const at::Tensor& t, const char* name) {
  TORCH_CHECK(t.is_cuda() && t.scalar_type() == at::kFloat && t.is_contiguous(), name, ": fp32 device tensor expected");
}
void chk_table(const at::Tensor& ptab) {
  TORCH_CHECK(ptab.is_cuda() && ptab.scalar_type() == at::kInt && ptab.dim() == 2 && ptab.stride(1) == 1,
              "page table: int32 [slots, pages]");
}

at::Tensor sm_embed(const at::Tensor& ids, const at::Tensor& table, double scale) {
  TORCH_CHECK(ids.is_cuda() && ids.scalar_type() == at::kLong && ids.is_contiguous() && ids.dim() == 1, "ids: int64 [T]");
  TORCH_CHECK(table.is_cuda() && table.dim() == 2 && table.is_contiguous() && is_act(table), "table: [V, W] fp32 / bf16");
  c10::hip::HIPGuardMasqueradingAsCUDA guard(table.device());
  auto out = at::empty({ids.size(0), table.size(1)}, table.options().dtype(at::kFloat));
  check(edge_sm_embed(ids.data_ptr<int64_t>(), table.data_ptr(), out.data_ptr<float>(), (int)ids.size(0),
                      (int)table.size(1), (int)table.size(0), (float)scale, f32(table), stream()), "sm_embed");
  return out;
}

at::Tensor sm_scalar_norm(const at::Tensor& x, const at::Tensor& gain, double eps, bool out_f32) {
  chk_f32(x, "x");
  chk_f32(gain, "gain");
  TORCH_CHECK(x.dim() == 2 && gain.numel() == 1, "x [T, W], gain [1]");
  c10::hip::HIPGuardMasqueradingAsCUDA guard(x.device());
  auto y = at::empty_like(x, x.options().dtype(act_type(out_f32)));
  check(edge_sm_scalar_norm(x.data_ptr<float>(), gain.data_ptr<float>(), y.data_ptr(), (int)x.size(0), (int)x.size(1),
                            (float)eps, out_f32, stream()), "sm_scalar_norm");
  return y;
}

at::Tensor sm_relu2(const at::Tensor& u, int64_t c0, int64_t C) {
  TORCH_CHECK(is_act(u), "u: fp32 / bf16");
  const int ld = row_ld(u, "u");
  TORCH_CHECK(c0 >= 0 && C >= 0 && c0 + C <= u.size(1), "columns out of range");
  c10::hip::HIPGuardMasqueradingAsCUDA guard(u.device());
  auto y = at::empty({u.size(0), C}, u.options());
  check(edge_sm_relu2(u.data_ptr(), ld, (int)c0, y.data_ptr(), (int)u.size(0), (int)C, f32(u), stream()), "sm_relu2");
  return y;
}

at::Tensor sm_cat_cast(const at::Tensor& a, const at::Tensor& b, bool out_f32) {
  chk_f32(a, "a");
  chk_f32(b, "b");
  TORCH_CHECK(a.dim() == 2 && a.sizes() == b.sizes(), "a, b: fp32 [T, W]");
  c10::hip::HIPGuardMasqueradingAsCUDA guard(a.device());
  auto y = at::empty({a.size(0), 2 * a.size(1)}, a.options().dtype(act_type(out_f32)));
  check(edge_sm_cat_cast(a.data_ptr<float>(), b.data_ptr<float>(), y.data_ptr(), (int)a.size(0), (int)a.size(1),
                         out_f32, stream()), "sm_cat_cast");
  return y;
}

void sm_combine(at::Tensor& x, const at::Tensor& l, const at::Tensor& r, const at::Tensor& wl, const at::Tensor& wr,
                double eps, const std::optional<at::Tensor>& extra) {
  chk_f32(x, "x");
  chk_f32(wl, "wl");
  chk_f32(wr, "wr");
  TORCH_CHECK(x.dim() == 2 && l.sizes() == x.sizes() && r.sizes() == x.sizes() && l.is_contiguous() &&
                  r.is_contiguous() && is_act(l) && r.scalar_type() == l.scalar_type() && l.is_cuda() && r.is_cuda(),
              "left / right: [T, W] like x");
  TORCH_CHECK(wl.numel() == x.size(1) && wr.numel() == x.size(1), "weights: [W]");
  if (extra) TORCH_CHECK(extra->sizes() == x.sizes() && extra->is_contiguous() && extra->is_cuda() &&
                             extra->scalar_type() == l.scalar_type(), "extra: [T, W] like left");
  c10::hip::HIPGuardMasqueradingAsCUDA guard(x.device());
  check(edge_sm_combine(x.data_ptr<float>(), l.data_ptr(), r.data_ptr(), wl.data_ptr<float>(), wr.data_ptr<float>(),
                        extra ? extra->data_ptr() : nullptr, (int)x.size(0), (int)x.size(1), (float)eps, f32(l),
                        stream()), "sm_combine");
}

at::Tensor sm_gated_norm(const at::Tensor& y, const at::Tensor& z, const at::Tensor& w, int64_t groups, double eps,
                         bool out_f32) {
  chk_f32(y, "y");
  chk_f32(w, "weight");
  const int z_ld = row_ld(z, "z");
  TORCH_CHECK(y.dim() == 2 && z.sizes() == y.sizes() && is_act(z) && f32(z) == (int)out_f32 && w.numel() == y.size(1),
              "y fp32 [T, C], z [T, C] in the output dtype, weight [C]");
  c10::hip::HIPGuardMasqueradingAsCUDA guard(y.device());
  auto out = at::empty_like(y, y.options().dtype(act_type(out_f32)));
  check(edge_sm_gated_norm(y.data_ptr<float>(), z.data_ptr(), z_ld, w.data_ptr<float>(), out.data_ptr(), (int)y.size(0),
                           (int)y.size(1), (int)groups, (float)eps, out_f32, stream()), "sm_gated_norm");
  return out;
}

at::Tensor sm_rope_write(const at::Tensor& proj, const at::Tensor& tok_seq, const at::Tensor& tok_pos,
                         const at::Tensor& seq_slot, const at::Tensor& ptab, const std::optional<at::Tensor>& rope,
                         at::Tensor& kp, const std::optional<at::Tensor>& vpo, int64_t H, int64_t rot) {
  const int ld = row_ld(proj, "proj");
  chk_i32(tok_seq, "tok_seq");
  chk_i32(tok_pos, "tok_pos");
  chk_i32(seq_slot, "seq_slot");
  chk_table(ptab);
  TORCH_CHECK(is_act(proj) && kp.scalar_type() == proj.scalar_type() && kp.is_cuda() && kp.is_contiguous() &&
                  kp.dim() == 4, "pages: [pages, page, G, D] in proj's dtype");
  const int64_t T = proj.size(0), page = kp.size(1), G = kp.size(2), D = kp.size(3);
  int64_t Dv = 0;                                            // no value pages: the keys are the values
  if (vpo) {
    const at::Tensor& vp = *vpo;
    TORCH_CHECK(vp.scalar_type() == proj.scalar_type() && vp.is_cuda() && vp.is_contiguous() && vp.dim() == 4 &&
                    vp.size(0) == kp.size(0) && vp.size(1) == page && vp.size(2) == G, "k / v pages differ");
    Dv = vp.size(3);
  }
  TORCH_CHECK(proj.size(1) == (H + G) * D + G * Dv, "proj: [T, (H + G) D + G Dv]");
  TORCH_CHECK(tok_seq.numel() == T && tok_pos.numel() == T, "token metadata: [T]");
  if (rot > 0) {
    TORCH_CHECK(rope && rope->is_cuda() && rope->scalar_type() == at::kFloat && rope->is_contiguous() &&
                    rope->dim() == 3 && rope->size(1) * 2 == rot && rope->size(2) == 2, "rope: fp32 [pos, rot/2, 2]");
  }
  c10::hip::HIPGuardMasqueradingAsCUDA guard(proj.device());
  auto q = at::empty({T, H, D}, proj.options());
  check(edge_sm_rope_write(proj.data_ptr(), ld, tok_seq.data_ptr<int>(), tok_pos.data_ptr<int>(),
                           seq_slot.data_ptr<int>(), ptab.data_ptr<int>(), (int)ptab.stride(0),
                           rot > 0 ? rope->data_ptr<float>() : nullptr, q.data_ptr(), kp.data_ptr(),
                           vpo ? vpo->data_ptr() : nullptr, (int)T,
                           (int)H, (int)G, (int)D, (int)Dv, (int)rot, (int)page, f32(proj), stream()), "sm_rope_write");
  return q;
}

void sm_pool_blocks(const at::Tensor& kp, const at::Tensor& vp, at::Tensor& kb, at::Tensor& vb,
                    const at::Tensor& seq_slot, const at::Tensor& seq_start, const at::Tensor& seq_len,
                    const at::Tensor& ptab, int64_t pool, int64_t n, int64_t max_blocks) {
  chk_i32(seq_slot, "seq_slot");
  chk_i32(seq_start, "seq_start");
  chk_i32(seq_len, "seq_len");
  chk_table(ptab);
  chk_f32(kb, "k_pool");
  chk_f32(vb, "v_pool");
  TORCH_CHECK(is_act(kp) && kp.is_cuda() && kp.is_contiguous() && vp.is_contiguous() && kp.dim() == 4 && vp.dim() == 4 &&
                  vp.scalar_type() == kp.scalar_type(), "pages: [pages, page, G, D]");
  const int64_t page = kp.size(1), G = kp.size(2), D = kp.size(3), Dv = vp.size(3);
  TORCH_CHECK(pool > 0 && kb.dim() == 4 && kb.size(0) == kp.size(0) && kb.size(1) == (page + pool - 1) / pool &&
                  kb.size(2) == G && kb.size(3) == D && vb.size(0) == kp.size(0) && vb.size(1) == kb.size(1) &&
                  vb.size(2) == G && vb.size(3) == Dv, "pooled entries: [pages, ceil(page / pool), G, D]");
  TORCH_CHECK(seq_slot.numel() >= n && seq_start.numel() >= n && seq_len.numel() >= n, "sequence metadata: [n]");
  c10::hip::HIPGuardMasqueradingAsCUDA guard(kp.device());
  check(edge_sm_pool_blocks(kp.data_ptr(), vp.data_ptr(), kb.data_ptr<float>(), vb.data_ptr<float>(),
                            seq_slot.data_ptr<int>(), seq_start.data_ptr<int>(), seq_len.data_ptr<int>(),
                            ptab.data_ptr<int>(), (int)ptab.stride(0), (int)n, (int)max_blocks, (int)G, (int)D, (int)Dv,
                            (int)page, (int)kb.size(1), (int)pool, f32(kp), stream()), "sm_pool_blocks");
}

at::Tensor sm_attention(const at::Tensor& q, const std::optional<at::Tensor>& gate, const at::Tensor& kp,
                        const at::Tensor& vp, const std::optional<at::Tensor>& kb, const std::optional<at::Tensor>& vb,
                        const at::Tensor& tok_seq, const at::Tensor& tok_pos, const at::Tensor& seq_slot,
                        const at::Tensor& ptab, double scale, int64_t window, int64_t pool, int64_t max_keys,
                        const std::optional<at::Tensor>& seq_start, const std::optional<at::Tensor>& seq_len,
                        const std::optional<at::Tensor>& seq_off, int64_t n, int64_t qtiles, bool chunked, double softcap,
                        const std::optional<at::Tensor>& slopes, const std::optional<at::Tensor>& sink,
                        int64_t keep_first) {
  // chunked: `window` is a chunk size and the gate is [T, H * Dv] (see attn_kernel); keep_first: the first
  // tokens of a sequence that stay visible behind a sliding window
  TORCH_CHECK(keep_first >= 0 && (keep_first == 0 || (window > 0 && !chunked)), "keep_first goes with a sliding window");
  chk_i32(tok_seq, "tok_seq");
  chk_i32(tok_pos, "tok_pos");
  chk_i32(seq_slot, "seq_slot");
  chk_table(ptab);
  TORCH_CHECK(q.is_cuda() && q.dim() == 3 && q.is_contiguous() && is_act(q), "q: [T, H, D]");
  TORCH_CHECK(kp.scalar_type() == q.scalar_type() && vp.scalar_type() == q.scalar_type() && kp.dim() == 4 &&
                  vp.dim() == 4 && kp.size(3) == q.size(2), "pages: [pages, page, G, D]");
  const int64_t T = q.size(0), H = q.size(1), D = q.size(2), page = kp.size(1), G = kp.size(2), Dv = vp.size(3);
  // rows of a page lie kld / vld elements apart (a value that is a slice of the key row shares its stride);
  // pages are dense runs of rows, heads dense inside a row
  const int64_t kld = kp.stride(1), vld = vp.stride(1);
  TORCH_CHECK(kp.stride(3) == 1 && vp.stride(3) == 1 && (G == 1 || (kp.stride(2) == D && vp.stride(2) == Dv)) &&
                  kp.stride(0) == page * kld && vp.stride(0) == page * vld && kld >= G * D && vld >= G * Dv &&
                  vp.size(0) == kp.size(0) && vp.size(1) == page && vp.size(2) == G, "pages: rows must be dense runs");
  TORCH_CHECK(max_keys <= ptab.size(1) * page, "page table too short for the step");
  int gate_ld = 0, PB = 0;
  if (gate) {
    gate_ld = row_ld(*gate, "gate");
    TORCH_CHECK(gate->size(0) == T && gate->size(1) == (chunked ? H * Dv : H) && gate->scalar_type() == q.scalar_type(),
                "gate: [T, H] (one per head) or [T, H Dv] (one per coordinate)");
  }
  const float* slopes_p = nullptr;
  const float* sink_p = nullptr;
  if (slopes) {
    chk_f32(*slopes, "slopes");
    TORCH_CHECK(slopes->numel() == H, "slopes: fp32 [H]");
    slopes_p = slopes->data_ptr<float>();
  }
  if (sink) {
    chk_f32(*sink, "sink");
    TORCH_CHECK(sink->numel() == H, "sink: fp32 [H]");
    sink_p = sink->data_ptr<float>();
  }
  TORCH_CHECK(!chunked || pool == 0, "chunked attention has no pooled blocks");
  const int gate_elem = chunked && gate ? 1 : 0;
  if (pool > 0 && window > 0) {
    TORCH_CHECK(kb && vb, "pooled entries missing");
    chk_f32(*kb, "k_pool");
    chk_f32(*vb, "v_pool");
    PB = (int)kb->size(1);
    TORCH_CHECK(kb->size(0) == kp.size(0) && PB == (page + pool - 1) / pool && kb->size(2) == G && kb->size(3) == D &&
                    vb->size(1) == PB && vb->size(3) == Dv, "pooled entries: [pages, ceil(page / pool), G, D]");
  }
  c10::hip::HIPGuardMasqueradingAsCUDA guard(q.device());
  auto out = at::empty({T, H * Dv}, q.options());
  if (qtiles > 0 && q.scalar_type() == at::kBFloat16) {
    // prompt portions in bf16 (qtiles = sum of ceil(len / 64)): the MFMA kernel when it takes the head sizes
    TORCH_CHECK(seq_start && seq_len && seq_off, "sequence metadata missing");
    chk_i32(*seq_start, "seq_start");
    chk_i32(*seq_len, "seq_len");
    chk_i32(*seq_off, "seq_off");
    TORCH_CHECK(seq_start->numel() >= n && seq_len->numel() >= n && seq_off->numel() >= n && seq_slot.numel() >= n &&
                    qtiles * 64 >= T, "sequence metadata: [n]");
    const int rc = edge_sm_attention_mfma(q.data_ptr(), gate ? gate->data_ptr() : nullptr, gate_ld, kp.data_ptr(),
                                          vp.data_ptr(), PB ? kb->data_ptr<float>() : nullptr,
                                          PB ? vb->data_ptr<float>() : nullptr, seq_slot.data_ptr<int>(),
                                          seq_start->data_ptr<int>(), seq_len->data_ptr<int>(), seq_off->data_ptr<int>(),
                                          ptab.data_ptr<int>(), (int)ptab.stride(0), out.data_ptr(), (int)n, (int)qtiles,
                                          (int)H, (int)G, (int)D, (int)Dv, (int)page, PB, (float)scale, (int)window,
                                          PB ? (int)pool : 0, (int)kld, (int)vld, chunked ? 1 : 0, (float)softcap, slopes_p,
                                          sink_p, gate_elem, (int)keep_first, stream());
    if (rc != 1) {
      check(rc, "sm_attention_mfma");
      return out;
    }
  }
  // few queries over many keys (decode steps): split every query's keys over several workgroups
  int nsplit = 1;
  {
    const int64_t vis = (window > 0 ? std::min<int64_t>(window + keep_first, max_keys) : max_keys) + (PB ? max_keys / pool : 0);
    const int64_t chunks = (vis + 255) / 256;
    if (T * G <= 64 && chunks > 1) nsplit = (int)std::min<int64_t>(chunks, 8);
  }
  at::Tensor part;
  if (nsplit > 1)
    part = at::empty({(int64_t)edge_sm_attention_part_floats((int)T, (int)H, (int)G, (int)D, (int)Dv, nsplit)},
                     q.options().dtype(at::kFloat));
  check(edge_sm_attention(q.data_ptr(), gate ? gate->data_ptr() : nullptr, gate_ld, kp.data_ptr(), vp.data_ptr(),
                          PB ? kb->data_ptr<float>() : nullptr, PB ? vb->data_ptr<float>() : nullptr,
                          tok_seq.data_ptr<int>(), tok_pos.data_ptr<int>(), seq_slot.data_ptr<int>(),
                          ptab.data_ptr<int>(), (int)ptab.stride(0), out.data_ptr(), (int)T, (int)H, (int)G, (int)D, (int)Dv,
                          (int)page, PB, (float)scale, (int)window, PB ? (int)pool : 0, f32(q), nsplit,
                          nsplit > 1 ? part.data_ptr<float>() : nullptr, (int)kld, (int)vld, chunked ? 1 : 0, (float)softcap,
                          slopes_p, sink_p, gate_elem, (int)keep_first, stream()), "sm_attention");
  return out;
}

at::Tensor sm_conv_silu(const at::Tensor& u, int64_t c0, int64_t C, const at::Tensor& w, const at::Tensor& bias,
                        at::Tensor& state, const at::Tensor& tok_seq, const at::Tensor& tok_pos,
                        const at::Tensor& seq_slot, const at::Tensor& seq_start, const at::Tensor& seq_len,
                        const at::Tensor& seq_off, int64_t n, int64_t max_len) {
  const int ld = row_ld(u, "u");
  chk_f32(w, "conv weight");
  chk_f32(bias, "conv bias");
  for (const at::Tensor* t : {&tok_seq, &tok_pos, &seq_slot, &seq_start, &seq_len, &seq_off}) chk_i32(*t, "metadata");
  const int64_t T = u.size(0), taps = w.size(1);
  TORCH_CHECK(is_act(u) && c0 >= 0 && c0 + C <= u.size(1) && w.dim() == 2 && w.size(0) == C && bias.numel() == C,
              "conv: weight [C, taps], bias [C], columns inside u");
  TORCH_CHECK(state.is_cuda() && state.is_contiguous() && state.scalar_type() == u.scalar_type() && state.dim() == 3 &&
                  state.size(1) == std::max<int64_t>(taps - 1, 1) && state.size(2) == C, "state: [slots, taps - 1, C]");
  TORCH_CHECK(tok_seq.numel() == T && tok_pos.numel() == T && seq_slot.numel() >= n, "metadata sizes");
  c10::hip::HIPGuardMasqueradingAsCUDA guard(u.device());
  auto out = at::empty({T, C}, u.options());
  check(edge_sm_conv_silu(u.data_ptr(), ld, (int)c0, (int)C, w.data_ptr<float>(), bias.data_ptr<float>(), state.data_ptr(),
                          tok_seq.data_ptr<int>(), tok_pos.data_ptr<int>(), seq_slot.data_ptr<int>(),
                          seq_start.data_ptr<int>(), seq_len.data_ptr<int>(), seq_off.data_ptr<int>(), out.data_ptr(),
                          (int)T, (int)n, (int)taps, f32(u), (int)max_len, stream()), "sm_conv_silu");
  return out;
}

at::Tensor sm_ssd_scan(const at::Tensor& xbc, const at::Tensor& u, int64_t dt0, const at::Tensor& dt_bias,
                       const at::Tensor& A_log, const at::Tensor& D, at::Tensor& state, const at::Tensor& seq_slot,
                       const at::Tensor& seq_start, const at::Tensor& seq_len, const at::Tensor& seq_off, int64_t n,
                       int64_t Hs, int64_t P, int64_t N, int64_t groups, int64_t chunks, int64_t max_chunks) {
  const int ld = row_ld(u, "u");
  chk_f32(dt_bias, "dt_bias");
  chk_f32(A_log, "A_log");
  chk_f32(D, "D");
  chk_f32(state, "state");
  for (const at::Tensor* t : {&seq_slot, &seq_start, &seq_len, &seq_off}) chk_i32(*t, "metadata");
  TORCH_CHECK(xbc.is_cuda() && xbc.is_contiguous() && xbc.dim() == 2 && is_act(xbc) &&
                  xbc.scalar_type() == u.scalar_type() && xbc.size(1) == Hs * P + 2 * groups * N &&
                  xbc.size(0) == u.size(0), "xbc: [T, inner + 2 groups N]");
  TORCH_CHECK(dt0 >= 0 && dt0 + Hs <= u.size(1) && dt_bias.numel() == Hs && A_log.numel() == Hs && D.numel() == Hs,
              "per-head constants: [heads]");
  TORCH_CHECK(state.dim() == 4 && state.size(1) == Hs && state.size(2) == N && state.size(3) == P,
              "state: fp32 [slots, heads, N, vdim]");
  TORCH_CHECK(seq_slot.numel() >= n && seq_start.numel() >= n && seq_len.numel() >= n && seq_off.numel() >= n,
              "sequence metadata: [n]");
  c10::hip::HIPGuardMasqueradingAsCUDA guard(xbc.device());
  auto y = at::empty({xbc.size(0), Hs * P}, xbc.options().dtype(at::kFloat));
  if (chunks > 0) {
    // long portions: the chunked form (chunks = sum of ceil(len / 64) over the step's sequences)
    TORCH_CHECK(chunks * 64 >= xbc.size(0) && max_chunks <= chunks, "chunk counts do not cover the step");
    auto sloc = at::empty({chunks, Hs, N, P}, y.options());
    auto cdec = at::empty({chunks, Hs}, y.options());
    check(edge_sm_ssd_chunked(xbc.data_ptr(), (int)xbc.size(1), u.data_ptr(), ld, (int)dt0, dt_bias.data_ptr<float>(),
                              A_log.data_ptr<float>(), D.data_ptr<float>(), state.data_ptr<float>(),
                              seq_slot.data_ptr<int>(), seq_start.data_ptr<int>(), seq_len.data_ptr<int>(),
                              seq_off.data_ptr<int>(), y.data_ptr<float>(), sloc.data_ptr<float>(), cdec.data_ptr<float>(),
                              (int)n, (int)max_chunks, (int)Hs, (int)P, (int)N, (int)groups, f32(xbc), stream()),
          "sm_ssd_chunked");
    return y;
  }
  check(edge_sm_ssd_scan(xbc.data_ptr(), (int)xbc.size(1), u.data_ptr(), ld, (int)dt0, dt_bias.data_ptr<float>(),
                         A_log.data_ptr<float>(), D.data_ptr<float>(), state.data_ptr<float>(), seq_slot.data_ptr<int>(),
                         seq_start.data_ptr<int>(), seq_len.data_ptr<int>(), seq_off.data_ptr<int>(), y.data_ptr<float>(),
                         (int)n, (int)Hs, (int)P, (int)N, (int)groups, f32(xbc), stream()), "sm_ssd_scan");
  return y;
}

// ---------------------------------------------------------------------------------- post-norm layers
void chk_act2(const at::Tensor& t, const char* name) {
  TORCH_CHECK(t.is_cuda() && t.dim() == 2 && t.is_contiguous() && is_act(t), name, ": contiguous fp32 / bf16 [rows, cols]");
}

at::Tensor sm_embed_bigram(const at::Tensor& ids, const at::Tensor& table, const at::Tensor& bigram, at::Tensor& prev_tok,
                           const at::Tensor& tok_seq, const at::Tensor& tok_pos, const at::Tensor& seq_slot,
                           const at::Tensor& seq_start, const at::Tensor& seq_len, const at::Tensor& seq_off, int64_t n,
                           int64_t buckets, int64_t mul_prev, int64_t mul_cur) {
  TORCH_CHECK(ids.is_cuda() && ids.scalar_type() == at::kLong && ids.is_contiguous() && ids.dim() == 1, "ids: int64 [T]");
  chk_act2(table, "table");
  chk_act2(bigram, "bigram");
  TORCH_CHECK(bigram.scalar_type() == table.scalar_type() && bigram.size(1) == table.size(1) && bigram.size(0) == buckets + 1,
              "bigram: [buckets + 1, W]");
  TORCH_CHECK(prev_tok.is_cuda() && prev_tok.scalar_type() == at::kLong && prev_tok.is_contiguous(), "prev_tok: int64 [slots]");
  for (const at::Tensor* t : {&tok_seq, &tok_pos, &seq_slot, &seq_start, &seq_len, &seq_off}) chk_i32(*t, "metadata");
  const int64_t T = ids.size(0);
  TORCH_CHECK(tok_seq.numel() == T && tok_pos.numel() == T && seq_slot.numel() >= n && seq_start.numel() >= n &&
                  seq_len.numel() >= n && seq_off.numel() >= n, "metadata sizes");
  c10::hip::HIPGuardMasqueradingAsCUDA guard(table.device());
  auto out = at::empty({T, table.size(1)}, table.options().dtype(at::kFloat));
  check(edge_sm_embed_bigram(ids.data_ptr<int64_t>(), table.data_ptr(), bigram.data_ptr(), prev_tok.data_ptr<int64_t>(),
                             tok_seq.data_ptr<int>(), tok_pos.data_ptr<int>(), seq_slot.data_ptr<int>(),
                             seq_start.data_ptr<int>(), seq_len.data_ptr<int>(), seq_off.data_ptr<int>(),
                             out.data_ptr<float>(), (int)T, (int)n, (int)table.size(1), (int)table.size(0), (long)buckets,
                             (long)mul_prev, (long)mul_cur, f32(table), stream()), "sm_embed_bigram");
  return out;
}

at::Tensor sm_canon(const at::Tensor& x, const at::Tensor& w, at::Tensor& state, const at::Tensor& tok_seq,
                    const at::Tensor& tok_pos, const at::Tensor& seq_slot, const at::Tensor& seq_start,
                    const at::Tensor& seq_len, const at::Tensor& seq_off, int64_t n, int64_t max_len, bool out_f32) {
  chk_f32(x, "x");
  chk_f32(w, "weight");
  chk_f32(state, "state");
  for (const at::Tensor* t : {&tok_seq, &tok_pos, &seq_slot, &seq_start, &seq_len, &seq_off}) chk_i32(*t, "metadata");
  TORCH_CHECK(x.dim() == 2 && w.dim() == 2 && w.size(0) == x.size(1), "x [T, W], weight [W, taps]");
  const int64_t T = x.size(0), W = x.size(1), taps = w.size(1);
  TORCH_CHECK(state.dim() == 3 && state.size(1) == std::max<int64_t>(taps - 1, 1) && state.size(2) == W,
              "state: fp32 [slots, taps - 1, W]");
  TORCH_CHECK(tok_seq.numel() == T && tok_pos.numel() == T && seq_slot.numel() >= n, "metadata sizes");
  c10::hip::HIPGuardMasqueradingAsCUDA guard(x.device());
  auto out = at::empty({T, W}, x.options().dtype(act_type(out_f32)));
  check(edge_sm_canon(x.data_ptr<float>(), (int)W, w.data_ptr<float>(), state.data_ptr<float>(), tok_seq.data_ptr<int>(),
                      tok_pos.data_ptr<int>(), seq_slot.data_ptr<int>(), seq_start.data_ptr<int>(), seq_len.data_ptr<int>(),
                      seq_off.data_ptr<int>(), out.data_ptr(), (int)T, (int)n, (int)taps, (int)max_len, out_f32, stream()),
        "sm_canon");
  return out;
}

at::Tensor sm_layer_norm(const at::Tensor& x, const at::Tensor& w, const at::Tensor& b, double eps, bool out_f32) {
  chk_f32(x, "x");
  chk_f32(w, "weight");
  chk_f32(b, "bias");
  TORCH_CHECK(x.dim() == 2 && w.numel() == x.size(1) && b.numel() == x.size(1), "x [T, W], weight / bias [W]");
  c10::hip::HIPGuardMasqueradingAsCUDA guard(x.device());
  auto y = at::empty_like(x, x.options().dtype(act_type(out_f32)));
  check(edge_sm_layer_norm(x.data_ptr<float>(), w.data_ptr<float>(), b.data_ptr<float>(), y.data_ptr(), (int)x.size(0),
                           (int)x.size(1), (float)eps, out_f32, stream()), "sm_layer_norm");
  return y;
}

void sm_ln_residual(at::Tensor& x, const std::optional<at::Tensor>& y, const at::Tensor& w, const at::Tensor& b, double eps,
                    const std::optional<at::Tensor>& parts, const std::optional<at::Tensor>& part_w) {
  chk_f32(x, "x");
  chk_f32(w, "weight");
  chk_f32(b, "bias");
  TORCH_CHECK(x.dim() == 2 && w.numel() == x.size(1) && b.numel() == x.size(1), "x [T, W], weight / bias [W]");
  TORCH_CHECK(y || parts, "nothing to norm");
  const int64_t T = x.size(0), W = x.size(1);
  int K = 0, is_f32 = 0;
  if (y) {
    chk_act2(*y, "y");
    TORCH_CHECK(y->size(0) == T && y->size(1) == W, "y: [T, W]");
    is_f32 = f32(*y);
  }
  if (parts) {
    TORCH_CHECK(part_w, "part weights missing");
    chk_f32(*part_w, "part weights");
    TORCH_CHECK(parts->is_cuda() && parts->is_contiguous() && is_act(*parts) && parts->dim() == 3 && parts->size(0) == T &&
                    parts->size(2) == W && part_w->dim() == 2 && part_w->size(0) == T && part_w->size(1) == parts->size(1) &&
                    (!y || parts->scalar_type() == y->scalar_type()), "parts [T, K, W], weights fp32 [T, K]");
    K = (int)parts->size(1);
    is_f32 = f32(*parts);
  }
  c10::hip::HIPGuardMasqueradingAsCUDA guard(x.device());
  check(edge_sm_ln_residual(x.data_ptr<float>(), y ? y->data_ptr() : nullptr, parts ? parts->data_ptr() : nullptr,
                            parts ? part_w->data_ptr<float>() : nullptr, K, w.data_ptr<float>(), b.data_ptr<float>(), (int)T,
                            (int)W, (float)eps, is_f32, stream()), "sm_ln_residual");
}

at::Tensor sm_rms_cols(const at::Tensor& u, int64_t c0, int64_t C, const at::Tensor& w, double eps, bool out_f32) {
  TORCH_CHECK(is_act(u) && (u.scalar_type() == at::kFloat) == out_f32, "u: fp32 / bf16, output of the same type");
  const int ld = row_ld(u, "u");
  chk_f32(w, "weight");
  TORCH_CHECK(c0 >= 0 && C > 0 && c0 + C <= u.size(1) && w.numel() == C, "columns out of range / weight [C]");
  c10::hip::HIPGuardMasqueradingAsCUDA guard(u.device());
  auto y = at::empty({u.size(0), C}, u.options());
  check(edge_sm_rms_cols(u.data_ptr(), ld, (int)c0, (int)C, w.data_ptr<float>(), y.data_ptr(), (int)u.size(0), (float)eps,
                         f32(u), stream()), "sm_rms_cols");
  return y;
}

at::Tensor sm_head_norm_gate(const at::Tensor& y, const at::Tensor& z, const at::Tensor& w, int64_t heads, double eps,
                             bool out_f32, bool silu) {
  chk_f32(y, "y");
  chk_f32(w, "weight");
  const int z_ld = row_ld(z, "z");
  TORCH_CHECK(y.dim() == 2 && heads > 0 && y.size(1) % heads == 0 && w.numel() == y.size(1) / heads && is_act(z) &&
                  z.size(0) == y.size(0) && z.size(1) == y.size(1) && (z.scalar_type() == at::kFloat) == out_f32,
              "y fp32 [T, heads P], z [T, heads P], weight [P]");
  c10::hip::HIPGuardMasqueradingAsCUDA guard(y.device());
  auto out = at::empty({y.size(0), y.size(1)}, z.options());
  check(edge_sm_head_norm_gate(y.data_ptr<float>(), z.data_ptr(), z_ld, w.data_ptr<float>(), out.data_ptr(), (int)y.size(0),
                               (int)heads, (int)(y.size(1) / heads), (float)eps, silu ? 1 : 0, f32(z), stream()),
        "sm_head_norm_gate");
  return out;
}

at::Tensor sm_glu_clamp(const at::Tensor& u, int64_t ff, double limit) {
  TORCH_CHECK(is_act(u), "u: fp32 / bf16");
  const int ld = row_ld(u, "u");
  TORCH_CHECK(ff >= 0 && 2 * ff <= u.size(1), "u: [T, gate | up]");
  c10::hip::HIPGuardMasqueradingAsCUDA guard(u.device());
  auto y = at::empty({u.size(0), ff}, u.options());
  check(edge_sm_glu_clamp(u.data_ptr(), ld, y.data_ptr(), (int)u.size(0), (int)ff, (float)limit, f32(u), stream()),
        "sm_glu_clamp");
  return y;
}

at::Tensor sm_latent_write(const std::optional<at::Tensor>& u, int64_t c0, const std::optional<at::Tensor>& w, double eps,
                           const at::Tensor& q, const at::Tensor& q_lat, const at::Tensor& tok_seq, const at::Tensor& tok_pos,
                           const at::Tensor& seq_slot, const at::Tensor& ptab, const std::optional<at::Tensor>& cs,
                           at::Tensor& pages, int64_t kvr, int64_t rot) {
  chk_i32(tok_seq, "tok_seq");
  chk_i32(tok_pos, "tok_pos");
  chk_i32(seq_slot, "seq_slot");
  chk_table(ptab);
  TORCH_CHECK(q.is_cuda() && q.dim() == 3 && q.is_contiguous() && is_act(q), "q: [T, H, D + R]");
  TORCH_CHECK(pages.is_cuda() && pages.is_contiguous() && pages.dim() == 4 && pages.size(2) == 1 &&
                  pages.scalar_type() == q.scalar_type() && pages.size(3) >= kvr, "pages: [pages, page, 1, kv_rank + R]");
  const int64_t T = q.size(0), H = q.size(1), R = pages.size(3) - kvr, D = q.size(2) - R, page = pages.size(1);
  TORCH_CHECK(D >= 0 && q_lat.is_cuda() && q_lat.dim() == 3 && q_lat.size(0) == T && q_lat.size(1) == H &&
                  q_lat.size(2) == kvr && q_lat.stride(2) == 1 && q_lat.scalar_type() == q.scalar_type(),
              "q_lat: [T, H, kv_rank], rows contiguous");
  TORCH_CHECK(tok_seq.numel() == T && tok_pos.numel() == T, "metadata sizes");
  int ld = 0;
  if (u) {
    ld = row_ld(*u, "u");
    TORCH_CHECK(w, "latent norm weight missing");
    chk_f32(*w, "latent norm weight");
    TORCH_CHECK(u->scalar_type() == q.scalar_type() && u->size(0) == T && c0 >= 0 && c0 + kvr + R <= u->size(1) &&
                    w->numel() == kvr, "u: [T, .. latent | key part ..]");
  }
  if (rot > 0) {
    TORCH_CHECK(cs, "rotary table missing");
    chk_f32(*cs, "rotary table");
    TORCH_CHECK(cs->dim() == 3 && cs->size(1) == rot / 2 && cs->size(2) == 2, "rotary table: [positions, rot / 2, 2]");
  }
  c10::hip::HIPGuardMasqueradingAsCUDA guard(q.device());
  auto qc = at::empty({T, H, kvr + R}, q.options());
  check(edge_sm_latent_write(u ? u->data_ptr() : nullptr, ld, (int)c0, u ? w->data_ptr<float>() : nullptr, (float)eps,
                             q.data_ptr(), q_lat.data_ptr(), (long)q_lat.stride(0), (long)q_lat.stride(1),
                             tok_seq.data_ptr<int>(), tok_pos.data_ptr<int>(), seq_slot.data_ptr<int>(), ptab.data_ptr<int>(),
                             (int)ptab.stride(0), rot > 0 ? cs->data_ptr<float>() : nullptr, pages.data_ptr(), qc.data_ptr(),
                             (int)T, (int)H, (int)D, (int)R, (int)kvr, (int)rot, (int)page, f32(q), stream()),
        "sm_latent_write");
  return qc;
}

at::Tensor sm_delta_prep(const at::Tensor& qkv, const at::Tensor& u, int64_t b0, const at::Tensor& a, const at::Tensor& dt_bias,
                         const at::Tensor& A_log, int64_t H, int64_t G, int64_t N) {
  chk_act2(qkv, "qkv");
  const int ld = row_ld(u, "u");
  chk_f32(a, "a");
  chk_f32(dt_bias, "dt_bias");
  chk_f32(A_log, "A_log");
  const int64_t T = qkv.size(0);
  TORCH_CHECK(u.scalar_type() == qkv.scalar_type() && u.size(0) == T && b0 >= 0 && b0 + H <= u.size(1) &&
                  qkv.size(1) >= 2 * G * N && a.dim() == 2 && a.size(0) == T && a.size(1) == H * N &&
                  dt_bias.numel() == H * N && A_log.numel() == H, "delta prep shapes");
  c10::hip::HIPGuardMasqueradingAsCUDA guard(qkv.device());
  auto prep = at::empty({T, 2 * G * N + H * N + H}, qkv.options().dtype(at::kFloat));
  check(edge_sm_delta_prep(qkv.data_ptr(), (int)qkv.size(1), u.data_ptr(), ld, (int)b0, a.data_ptr<float>(),
                           dt_bias.data_ptr<float>(), A_log.data_ptr<float>(), prep.data_ptr<float>(), (int)T, (int)H,
                           (int)G, (int)N, f32(qkv), stream()), "sm_delta_prep");
  return prep;
}

at::Tensor sm_delta_scan(const at::Tensor& prep, const at::Tensor& qkv, at::Tensor& state, const at::Tensor& seq_slot,
                         const at::Tensor& seq_start, const at::Tensor& seq_len, const at::Tensor& seq_off, int64_t n,
                         int64_t H, int64_t G, int64_t N, int64_t P) {
  chk_f32(prep, "prep");
  chk_f32(state, "state");
  chk_act2(qkv, "qkv");
  for (const at::Tensor* t : {&seq_slot, &seq_start, &seq_len, &seq_off}) chk_i32(*t, "metadata");
  const int64_t T = qkv.size(0);
  // a decay per head and key channel (H N numbers a row) or one per head (H numbers)
  TORCH_CHECK(prep.dim() == 2 && prep.size(0) == T &&
                  (prep.size(1) == 2 * G * N + H * N + H || prep.size(1) == 2 * G * N + 2 * H) &&
                  qkv.size(1) == 2 * G * N + H * P, "prep [T, q | k | decay | beta], qkv [T, q | k | v]");
  const int GD = prep.size(1) == 2 * G * N + H * N + H ? (int)N : 1;
  TORCH_CHECK(state.dim() == 4 && state.size(1) == H && state.size(2) == N && state.size(3) == P,
              "state: fp32 [slots, heads, N, P]");
  TORCH_CHECK(seq_slot.numel() >= n && seq_start.numel() >= n && seq_len.numel() >= n && seq_off.numel() >= n,
              "sequence metadata: [n]");
  c10::hip::HIPGuardMasqueradingAsCUDA guard(qkv.device());
  auto y = at::empty({T, H * P}, prep.options());
  check(edge_sm_delta_scan(prep.data_ptr<float>(), (int)prep.size(1), qkv.data_ptr(), (int)qkv.size(1), state.data_ptr<float>(),
                           seq_slot.data_ptr<int>(), seq_start.data_ptr<int>(), seq_len.data_ptr<int>(),
                           seq_off.data_ptr<int>(), y.data_ptr<float>(), (int)n, (int)H, (int)G, (int)N, (int)P, GD,
                           f32(qkv), stream()), "sm_delta_scan");
  return y;
}

// mode 0: softmax over all experts, the chosen ones renormalised; 1: sigmoid scores; 2: softmax over the chosen logits
std::tuple<at::Tensor, at::Tensor> sm_moe_route(const at::Tensor& h, const at::Tensor& router, int64_t top, double scale,
                                                int64_t mode, const std::optional<at::Tensor>& bias) {
  chk_act2(h, "h");
  chk_f32(router, "router");
  TORCH_CHECK(router.dim() == 2 && router.size(1) == h.size(1) && mode >= 0 && mode <= 2, "router: fp32 [E, W]");
  if (bias) {
    chk_f32(*bias, "bias");
    TORCH_CHECK(bias->numel() == router.size(0), "bias: fp32 [E]");
  }
  c10::hip::HIPGuardMasqueradingAsCUDA guard(h.device());
  auto idx = at::empty({h.size(0), top}, h.options().dtype(at::kInt));
  auto wts = at::empty({h.size(0), top}, h.options().dtype(at::kFloat));
  auto z = at::empty({h.size(0), router.size(0)}, wts.options());
  check(edge_sm_moe_route(h.data_ptr(), (int)h.size(1), router.data_ptr<float>(), bias ? bias->data_ptr<float>() : nullptr,
                          (int)router.size(0), (int)top, (float)scale, z.data_ptr<float>(), idx.data_ptr<int>(),
                          wts.data_ptr<float>(), (int)h.size(0), (int)mode, f32(h), stream()), "sm_moe_route");
  return {idx, wts};
}

at::Tensor sm_moe_experts(const at::Tensor& h, const at::Tensor& idx, const at::Tensor& w_gu, const at::Tensor& w_down,
                          double limit, bool silu, const std::optional<at::Tensor>& in_w) {
  chk_act2(h, "h");
  chk_i32(idx, "idx");
  const int64_t T = h.size(0), W = h.size(1);
  TORCH_CHECK(idx.dim() == 2 && idx.size(0) == T, "idx: int32 [T, top]");
  TORCH_CHECK(w_gu.is_cuda() && w_gu.is_contiguous() && w_gu.dim() == 3 && w_gu.size(2) == W && w_gu.size(1) % 2 == 0 &&
                  w_down.is_cuda() && w_down.is_contiguous() && w_down.dim() == 3 && w_down.size(0) == w_gu.size(0) &&
                  w_down.size(1) == W && w_down.size(2) == w_gu.size(1) / 2 && w_gu.scalar_type() == h.scalar_type() &&
                  w_down.scalar_type() == h.scalar_type(), "experts: w_gu [E, 2 ff, W], w_down [E, W, ff]");
  const int64_t top = idx.size(1), ff = w_gu.size(1) / 2;
  if (in_w) {
    chk_f32(*in_w, "in_w");
    TORCH_CHECK(silu && in_w->numel() == T * top, "in_w: fp32 [T, top], with the silu unit only");
  }
  c10::hip::HIPGuardMasqueradingAsCUDA guard(h.device());
  auto y = at::empty({T * top, ff}, h.options());
  auto out = at::empty({T, top, W}, h.options());
  check(edge_sm_moe_experts(h.data_ptr(), (int)W, idx.data_ptr<int>(), (int)top, w_gu.data_ptr(), w_down.data_ptr(), (int)ff,
                            (float)limit, silu ? 1 : 0, in_w ? in_w->data_ptr<float>() : nullptr, y.data_ptr(),
                            out.data_ptr(), (int)T, (int)w_gu.size(0), f32(h), stream()),
        "sm_moe_experts");
  return out;
}

at::Tensor sm_group_norm(const at::Tensor& x, const at::Tensor& w, int64_t groups, double eps, bool out_f32) {
  chk_f32(x, "x");
  chk_f32(w, "weight");
  TORCH_CHECK(x.dim() == 2 && w.numel() == x.size(1) && groups > 0 && x.size(1) % groups == 0,
              "x fp32 [T, W], weight [W], W a multiple of groups");
  c10::hip::HIPGuardMasqueradingAsCUDA guard(x.device());
  auto y = at::empty({x.size(0), x.size(1)}, x.options().dtype(act_type(out_f32)));
  check(edge_sm_group_norm(x.data_ptr<float>(), w.data_ptr<float>(), y.data_ptr(), (int)x.size(0), (int)x.size(1),
                           (int)groups, (float)eps, out_f32, stream()), "sm_group_norm");
  return y;
}

void sm_group_norm_residual(at::Tensor& x, const std::optional<at::Tensor>& y, const at::Tensor& w, int64_t groups,
                            double eps, double mult, const std::optional<at::Tensor>& parts,
                            const std::optional<at::Tensor>& part_w) {
  chk_f32(x, "x");
  chk_f32(w, "weight");
  TORCH_CHECK(x.dim() == 2 && w.numel() == x.size(1) && groups > 0 && x.size(1) % groups == 0 && (y || parts),
              "x fp32 [T, W], weight [W], W a multiple of groups, y or parts");
  const int64_t T = x.size(0), W = x.size(1);
  int is_f32 = 0, K = 0;
  if (y) {
    chk_act2(*y, "y");
    TORCH_CHECK(y->size(0) == T && y->size(1) == W, "y: [T, W]");
    is_f32 = f32(*y);
  }
  if (parts) {
    TORCH_CHECK(parts->is_cuda() && parts->is_contiguous() && is_act(*parts) && parts->dim() == 3 && parts->size(0) == T &&
                    parts->size(2) == W && (!y || parts->scalar_type() == y->scalar_type()), "parts: [T, K, W]");
    K = (int)parts->size(1);
    is_f32 = f32(*parts);
    if (part_w) {
      chk_f32(*part_w, "part_w");
      TORCH_CHECK(part_w->numel() == T * K, "part_w: fp32 [T, K]");
    }
  }
  c10::hip::HIPGuardMasqueradingAsCUDA guard(x.device());
  check(edge_sm_group_norm_residual(x.data_ptr<float>(), y ? y->data_ptr() : nullptr, parts ? parts->data_ptr() : nullptr,
                                    parts && part_w ? part_w->data_ptr<float>() : nullptr, K, w.data_ptr<float>(), (int)T,
                                    (int)W, (int)groups, (float)eps, (float)mult, is_f32, stream()),
        "sm_group_norm_residual");
}

at::Tensor sm_glu_silu(const at::Tensor& u, int64_t ff, const std::optional<at::Tensor>& row_w) {
  TORCH_CHECK(is_act(u), "u: fp32 / bf16");
  const int ld = row_ld(u, "u");
  TORCH_CHECK(ff >= 0 && 2 * ff <= u.size(1), "u: [T, gate | up]");
  if (row_w) {
    chk_f32(*row_w, "row_w");
    TORCH_CHECK(row_w->numel() == u.size(0), "row_w: fp32 [T]");
  }
  c10::hip::HIPGuardMasqueradingAsCUDA guard(u.device());
  auto y = at::empty({u.size(0), ff}, u.options());
  check(edge_sm_glu_silu(u.data_ptr(), ld, y.data_ptr(), row_w ? row_w->data_ptr<float>() : nullptr, (int)u.size(0),
                         (int)ff, f32(u), stream()), "sm_glu_silu");
  return y;
}

at::Tensor sm_delta_prep_head(const at::Tensor& qkv, const at::Tensor& u, int64_t b0, int64_t a0, const at::Tensor& dt_bias,
                              const at::Tensor& A_log, int64_t H, int64_t G, int64_t N) {
  chk_act2(qkv, "qkv");
  const int ld = row_ld(u, "u");
  chk_f32(dt_bias, "dt_bias");
  chk_f32(A_log, "A_log");
  const int64_t T = qkv.size(0);
  TORCH_CHECK(u.scalar_type() == qkv.scalar_type() && u.size(0) == T && b0 >= 0 && b0 + H <= u.size(1) && a0 >= 0 &&
                  a0 + H <= u.size(1) && qkv.size(1) >= 2 * G * N && dt_bias.numel() == H && A_log.numel() == H &&
                  G > 0 && H % G == 0, "delta prep shapes");
  c10::hip::HIPGuardMasqueradingAsCUDA guard(qkv.device());
  auto prep = at::empty({T, 2 * G * N + 2 * H}, qkv.options().dtype(at::kFloat));
  check(edge_sm_delta_prep_head(qkv.data_ptr(), (int)qkv.size(1), u.data_ptr(), ld, (int)b0, (int)a0,
                                dt_bias.data_ptr<float>(), A_log.data_ptr<float>(), prep.data_ptr<float>(), (int)T, (int)H,
                                (int)G, (int)N, f32(qkv), stream()), "sm_delta_prep_head");
  return prep;
}

// ---------------------------------------------------------------------------------- residual streams, gated attention
at::Tensor sm_hyper_read_norm(const at::Tensor& X, const std::optional<at::Tensor>& in_w, const at::Tensor& w, double eps,
                              bool out_f32) {
  chk_f32(X, "X");
  chk_f32(w, "weight");
  TORCH_CHECK(X.dim() == 3 && w.numel() == X.size(2), "X fp32 [T, S, W], weight [W]");
  if (in_w) {
    chk_f32(*in_w, "in_w");
    TORCH_CHECK(in_w->numel() == X.size(1), "in_w: fp32 [S]");
  }
  c10::hip::HIPGuardMasqueradingAsCUDA guard(X.device());
  auto y = at::empty({X.size(0), X.size(2)}, X.options().dtype(act_type(out_f32)));
  check(edge_sm_hyper_read_norm(X.data_ptr<float>(), in_w ? in_w->data_ptr<float>() : nullptr, w.data_ptr<float>(),
                                y.data_ptr(), (int)X.size(0), (int)X.size(1), (int)X.size(2), (float)eps, out_f32, stream()),
        "sm_hyper_read_norm");
  return y;
}

// next_w given: also returns the next sublayer's input, norm(sum_r next_in[r] X_new[:, r]) next_w, in the dtype of y / parts
std::optional<at::Tensor> sm_hyper_update(at::Tensor& X, const std::optional<at::Tensor>& mix,
                                          const std::optional<at::Tensor>& out_w, const std::optional<at::Tensor>& y,
                                          const std::optional<at::Tensor>& parts, const std::optional<at::Tensor>& part_w,
                                          const std::optional<at::Tensor>& next_in, const std::optional<at::Tensor>& next_w,
                                          double eps) {
  chk_f32(X, "X");
  TORCH_CHECK(X.dim() == 3 && (y || parts) && bool(mix) == bool(out_w), "X fp32 [T, S, W]; y or parts; mix with out_w");
  const int64_t T = X.size(0), S = X.size(1), W = X.size(2);
  if (mix) {
    chk_f32(*mix, "mix");
    chk_f32(*out_w, "out_w");
    TORCH_CHECK(mix->numel() == S * S && out_w->numel() == S, "mix fp32 [S, S], out_w fp32 [S]");
  }
  int is_f32 = 0, K = 0;
  if (y) {
    chk_act2(*y, "y");
    TORCH_CHECK(y->size(0) == T && y->size(1) == W, "y: [T, W]");
    is_f32 = f32(*y);
  }
  if (parts) {
    TORCH_CHECK(parts->is_cuda() && parts->is_contiguous() && is_act(*parts) && parts->dim() == 3 && parts->size(0) == T &&
                    parts->size(2) == W && (!y || parts->scalar_type() == y->scalar_type()), "parts: [T, K, W]");
    K = (int)parts->size(1);
    is_f32 = f32(*parts);
    if (part_w) {
      chk_f32(*part_w, "part_w");
      TORCH_CHECK(part_w->numel() == T * K, "part_w: fp32 [T, K]");
    }
  }
  c10::hip::HIPGuardMasqueradingAsCUDA guard(X.device());
  std::optional<at::Tensor> h;
  if (next_w) {
    chk_f32(*next_w, "next_w");
    TORCH_CHECK(next_w->numel() == W, "next_w: fp32 [W]");
    if (next_in) {
      chk_f32(*next_in, "next_in");
      TORCH_CHECK(next_in->numel() == S, "next_in: fp32 [S]");
    }
    h = at::empty({T, W}, X.options().dtype(act_type(is_f32)));
  }
  check(edge_sm_hyper_update(X.data_ptr<float>(), mix ? mix->data_ptr<float>() : nullptr,
                             out_w ? out_w->data_ptr<float>() : nullptr, y ? y->data_ptr() : nullptr,
                             parts ? parts->data_ptr() : nullptr, parts && part_w ? part_w->data_ptr<float>() : nullptr, K,
                             (int)T, (int)S, (int)W, (h && next_in) ? next_in->data_ptr<float>() : nullptr,
                             h ? next_w->data_ptr<float>() : nullptr, h ? h->data_ptr() : nullptr, (float)eps, is_f32,
                             stream()), "sm_hyper_update");
  return h;
}

at::Tensor sm_poly_norm(const at::Tensor& z, const at::Tensor& coef, double eps) {
  TORCH_CHECK(is_act(z), "z: fp32 / bf16");
  const int ld = row_ld(z, "z");
  chk_f32(coef, "coef");
  TORCH_CHECK(coef.numel() == 4, "coef: fp32 [4]");
  c10::hip::HIPGuardMasqueradingAsCUDA guard(z.device());
  auto y = at::empty({z.size(0), z.size(1)}, z.options());
  check(edge_sm_poly_norm(z.data_ptr(), ld, coef.data_ptr<float>(), y.data_ptr(), (int)z.size(0), (int)z.size(1), (float)eps,
                          f32(z), stream()), "sm_poly_norm");
  return y;
}

at::Tensor sm_qk_norm_rope_write(const at::Tensor& proj, const at::Tensor& tok_seq, const at::Tensor& tok_pos,
                                 const at::Tensor& seq_slot, const at::Tensor& ptab, const std::optional<at::Tensor>& qw,
                                 const std::optional<at::Tensor>& kw, double eps, const std::optional<at::Tensor>& rope,
                                 const std::optional<at::Tensor>& vrope, const std::optional<at::Tensor>& temp,
                                 at::Tensor& kp, at::Tensor& vp, int64_t H, int64_t rot) {
  const int ld = row_ld(proj, "proj");
  chk_i32(tok_seq, "tok_seq");
  chk_i32(tok_pos, "tok_pos");
  chk_i32(seq_slot, "seq_slot");
  chk_table(ptab);
  TORCH_CHECK(is_act(proj) && kp.scalar_type() == proj.scalar_type() && kp.is_cuda() && kp.is_contiguous() && kp.dim() == 4 &&
                  vp.scalar_type() == proj.scalar_type() && vp.is_cuda() && vp.is_contiguous() && vp.dim() == 4 &&
                  vp.size(0) == kp.size(0) && vp.size(1) == kp.size(1) && vp.size(2) == kp.size(2),
              "pages: [pages, page, G, D] and [pages, page, G, Dv] in proj's dtype");
  const int64_t T = proj.size(0), page = kp.size(1), G = kp.size(2), D = kp.size(3), Dv = vp.size(3);
  TORCH_CHECK(proj.size(1) >= (H + G) * D + G * Dv, "proj: [T, (H + G) D + G Dv + ..]");
  TORCH_CHECK(tok_seq.numel() == T && tok_pos.numel() == T, "token metadata: [T]");
  auto table = [&](const std::optional<at::Tensor>& t, int64_t dims, const char* name) -> const float* {
    if (!t) return nullptr;
    TORCH_CHECK(t->is_cuda() && t->scalar_type() == at::kFloat && t->is_contiguous() && t->dim() == 3 &&
                    t->size(1) * 2 == dims && t->size(2) == 2, name, ": fp32 [pos, dims / 2, 2]");
    return t->data_ptr<float>();
  };
  auto vec = [&](const std::optional<at::Tensor>& t, int64_t n, const char* name) -> const float* {
    if (!t) return nullptr;
    chk_f32(*t, name);
    TORCH_CHECK(t->numel() == n, name, ": wrong size");
    return t->data_ptr<float>();
  };
  TORCH_CHECK(rot == 0 || rope, "rope table missing");
  const float* cs = rot > 0 ? table(rope, rot, "rope") : nullptr;
  const float* vcs = table(vrope, Dv, "value rope");
  c10::hip::HIPGuardMasqueradingAsCUDA guard(proj.device());
  auto q = at::empty({T, H, D}, proj.options());
  check(edge_sm_qk_norm_rope_write(proj.data_ptr(), ld, tok_seq.data_ptr<int>(), tok_pos.data_ptr<int>(),
                                   seq_slot.data_ptr<int>(), ptab.data_ptr<int>(), (int)ptab.stride(0), vec(qw, D, "q norm"),
                                   vec(kw, D, "k norm"), (float)eps, cs, vcs, vec(temp, H, "temp"), q.data_ptr(),
                                   kp.data_ptr(), vp.data_ptr(), (int)T, (int)H, (int)G, (int)D, (int)Dv, (int)rot, (int)page,
                                   f32(proj), stream()), "sm_qk_norm_rope_write");
  return q;
}

at::Tensor sm_unrotate_gate(const at::Tensor& a, const std::optional<at::Tensor>& gate, const at::Tensor& tok_pos,
                            const std::optional<at::Tensor>& vrope, int64_t H) {
  chk_act2(a, "a");
  chk_i32(tok_pos, "tok_pos");
  const int64_t T = a.size(0), HD = a.size(1);
  TORCH_CHECK(H > 0 && HD % H == 0 && tok_pos.numel() == T, "a: [T, H Dv], tok_pos [T]");
  const int64_t Dv = HD / H;
  int gate_ld = 0;
  if (gate) {
    gate_ld = row_ld(*gate, "gate");
    TORCH_CHECK(gate->size(0) == T && gate->size(1) == HD && gate->scalar_type() == a.scalar_type(), "gate: [T, H Dv]");
  }
  if (vrope)
    TORCH_CHECK(vrope->is_cuda() && vrope->scalar_type() == at::kFloat && vrope->is_contiguous() && vrope->dim() == 3 &&
                    vrope->size(1) * 2 == Dv && vrope->size(2) == 2, "value rope: fp32 [pos, Dv / 2, 2]");
  c10::hip::HIPGuardMasqueradingAsCUDA guard(a.device());
  auto out = at::empty_like(a);
  check(edge_sm_unrotate_gate(a.data_ptr(), gate ? gate->data_ptr() : nullptr, gate_ld, tok_pos.data_ptr<int>(),
                              vrope ? vrope->data_ptr<float>() : nullptr, out.data_ptr(), (int)T, (int)HD, (int)Dv, f32(a),
                              stream()), "sm_unrotate_gate");
  return out;
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.def("sm_embed", &sm_embed);
  m.def("sm_scalar_norm", &sm_scalar_norm);
  m.def("sm_relu2", &sm_relu2);
  m.def("sm_cat_cast", &sm_cat_cast);
  m.def("sm_combine", &sm_combine);
  m.def("sm_gated_norm", &sm_gated_norm);
  m.def("sm_rope_write", &sm_rope_write);
  m.def("sm_pool_blocks", &sm_pool_blocks);
  m.def("sm_attention", &sm_attention);
  m.def("sm_conv_silu", &sm_conv_silu);
  m.def("sm_ssd_scan", &sm_ssd_scan);
  m.def("sm_embed_bigram", &sm_embed_bigram);
  m.def("sm_canon", &sm_canon);
  m.def("sm_layer_norm", &sm_layer_norm);
  m.def("sm_ln_residual", &sm_ln_residual);
  m.def("sm_rms_cols", &sm_rms_cols);
  m.def("sm_head_norm_gate", &sm_head_norm_gate);
  m.def("sm_glu_clamp", &sm_glu_clamp);
  m.def("sm_latent_write", &sm_latent_write);
  m.def("sm_delta_prep", &sm_delta_prep);
  m.def("sm_delta_scan", &sm_delta_scan);
  m.def("sm_moe_route", &sm_moe_route);
  m.def("sm_moe_experts", &sm_moe_experts);
  m.def("sm_group_norm", &sm_group_norm);
  m.def("sm_group_norm_residual", &sm_group_norm_residual);
  m.def("sm_glu_silu", &sm_glu_silu);
  m.def("sm_delta_prep_head", &sm_delta_prep_head);
  m.def("sm_hyper_read_norm", &sm_hyper_read_norm);
  m.def("sm_hyper_update", &sm_hyper_update);
  m.def("sm_poly_norm", &sm_poly_norm);
  m.def("sm_qk_norm_rope_write", &sm_qk_norm_rope_write);
  m.def("sm_unrotate_gate", &sm_unrotate_gate);
}
