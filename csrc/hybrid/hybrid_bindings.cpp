// pybind11 bindings of the grouped-attention + recurrence family (module theroundtaible_amd._C_hybrid):
// torch tensors -> raw HIP launchers on the current HIP stream, so every kernel can be captured by
// a hipGraph like any torch op. Every entry point validates dtype / device / contiguity / shape
// BEFORE launching: a hand-written kernel never sees operands its grid does not assume.
#include <torch/extension.h>
#include <c10/hip/HIPStream.h>
#include <hip/hip_runtime.h>

void launch_shift_norm(void* out, float* xs, const float* x, const void* y, const float* w, const float* mu,
                       float* state, const int* row_seq, const int64_t* positions, const int* start_pos,
                       const int* slots, int T, int W, int groups, int n_mix, float eps, bool out_bf, bool y_bf,
                       bool store_state, hipStream_t stream);
void launch_shift_state(const float* x, const float* w, float* state, const int* cu_q, const int* slots, int S, int W,
                        int groups, float eps, hipStream_t stream);
void launch_qk_prep(void* q, const void* proj, int stride, int q_off, int k_off, int v_off, bool v_from_k,
                    const float* inv_freq, int rot_dims, float eps, const int64_t* positions, void* kc, void* vc,
                    const int64_t* slot_mapping, int T, int H, int G, int Dk, int Dv, int BS, bool bf, int layout,
                    const float* q_scale, const float* q_w, const float* k_w, bool v_norm, float qt_coef, int qt_every,
                    hipStream_t stream);
void launch_mingru_scan(void* out, const void* proj, int stride, int z_off, int x_off, int g_off, int width,
                        const float* bz, const float* bx, float* state, const int* cu_q, const int* start_pos,
                        const int* slots, int S, bool bf, hipStream_t stream);
int mingru_scan_chunk();
void launch_mingru_chunked(void* out, const void* proj, int stride, int z_off, int x_off, int g_off, int width,
                           const float* bz, const float* bx, float* state, const int* cu_q, const int* start_pos,
                           const int* slots, int S, const int* chunks, int n_chunks, const int* seq_chunk0, float* ws,
                           bool bf, hipStream_t stream);
void launch_dual_norm_add(float* x, const void* a, const float* wa, const void* b, const float* wb, int T, int W,
                          float eps, bool bf, hipStream_t stream);
void launch_add_norm(void* out, float* x, const void* y, const float* w, int T, int W, int groups, float eps,
                     bool out_bf, bool y_bf, hipStream_t stream);
void launch_limited_glu(void* out, const void* gu, int64_t rows, int F, float limit, bool bf, hipStream_t stream);
int gqa_key_tile(int Dk, int Dv);
int launch_gqa_attention(void* out, const void* q, const void* kc, const void* vc, const int* block_tables,
                         const int* cu_q, const int* start_pos, const int* tiles, int n_tiles, const float* temp,
                         float* part_o, float* part_ml, int T, int H, int G, int Dk, int Dv, int BS, int max_blocks,
                         int rows, int num_splits, float scale, float sink, int window, const float* slopes,
                         const void* gate, int gate_stride, int layout, bool bf, hipStream_t stream);
int wkv_scan_chunk();
int launch_wkv_scan(void* out, const void* r, const void* k, const void* v, const void* g, const void* lw, int stride,
                    int lw_stride, const float* w0, const float* u, const float* norm_w, float* state, const int* cu_q,
                    const int* start_pos, const int* slots, int S, int H, int D, float eps, const int* chunks,
                    int n_chunks, const int* seq_chunk0, float* ws, bool bf, hipStream_t stream);
void launch_xielu(void* out, const void* a, const float* bias, int64_t rows, int F, float ap, float an, bool bf,
                  hipStream_t stream);
void launch_silu_glu(void* out, const void* gu, int64_t rows, int F, bool bf, hipStream_t stream);
int launch_topk_softmax(int* idx, float* wt, const float* logits, int T, int E, int top, hipStream_t stream);
int launch_moe_rows(void* out, float* hid, const void* h, const void* wgu, const void* wd, const int* idx,
                    const float* wt, int T, int W, int F, int top, bool bf, hipStream_t stream);

namespace {

hipStream_t cur() { return c10::hip::getCurrentHIPStream().stream(); }

bool is_bf(const torch::Tensor& t) { return t.scalar_type() == torch::kBFloat16; }

void chk(const torch::Tensor& t, const char* name) {
  TORCH_CHECK(t.is_cuda(), name, " must be a GPU tensor");
  TORCH_CHECK(t.is_contiguous(), name, " must be contiguous");
}
void chk_act(const torch::Tensor& t, const char* name) {
  chk(t, name);
  TORCH_CHECK(is_bf(t) || t.scalar_type() == torch::kFloat32, name, " must be bf16 or fp32");
}
void chk_f32(const torch::Tensor& t, const char* name, int64_t n = -1) {
  chk(t, name);
  TORCH_CHECK(t.scalar_type() == torch::kFloat32, name, " must be fp32");
  TORCH_CHECK(n < 0 || t.numel() == n, name, " has ", t.numel(), " entries, expected ", n);
}
void chk_i32(const torch::Tensor& t, const char* name, int64_t n = -1) {
  chk(t, name);
  TORCH_CHECK(t.scalar_type() == torch::kInt32, name, " must be int32");
  TORCH_CHECK(n < 0 || t.numel() == n, name, " has ", t.numel(), " entries, expected ", n);
}
void chk_i64(const torch::Tensor& t, const char* name, int64_t n) {
  chk(t, name);
  TORCH_CHECK(t.scalar_type() == torch::kInt64 && t.numel() == n, name, " must be int64 [", n, "]");
}

void shift_norm(torch::Tensor out, torch::Tensor xs, torch::Tensor x, c10::optional<torch::Tensor> y, torch::Tensor w,
                double eps, torch::Tensor mu, torch::Tensor state, torch::Tensor row_seq, torch::Tensor positions,
                torch::Tensor start_pos, torch::Tensor slots, bool store_state, int64_t groups) {
  chk_act(out, "out"); chk_f32(xs, "xs"); chk_f32(x, "x");
  TORCH_CHECK(x.dim() == 2 && xs.sizes() == x.sizes(), "shift_norm: shapes");
  const int64_t T = x.size(0), W = x.size(1);
  // out [T, W] for one mix, [n_mix, T, W] for several (mu [n_mix, W])
  const int64_t n_mix = out.dim() == 3 ? out.size(0) : 1;
  TORCH_CHECK(out.numel() == n_mix * T * W && out.size(-1) == W && out.size(-2) == T, "shift_norm: out [n_mix, T, W]");
  TORCH_CHECK(groups >= 1 && W % groups == 0, "shift_norm: the width must split into the norm groups");
  chk_f32(w, "w", W); chk_f32(mu, "mu", n_mix * W); chk_f32(state, "state");
  TORCH_CHECK(state.dim() == 2 && state.size(1) == W, "shift_norm: state must be [slots, W]");
  chk_i32(row_seq, "row_seq", T); chk_i64(positions, "positions", T);
  chk_i32(start_pos, "start_pos"); chk_i32(slots, "slots", start_pos.numel());
  const void* yp = nullptr;
  bool y_bf = false;
  if (y.has_value()) {
    chk_act(*y, "y");
    TORCH_CHECK(y->sizes() == x.sizes(), "shift_norm: y must have x's shape");
    TORCH_CHECK(xs.data_ptr() != x.data_ptr(), "shift_norm: with y the sum goes to a tensor of its own");
    yp = y->data_ptr();
    y_bf = is_bf(*y);
  }
  launch_shift_norm(out.data_ptr(), xs.data_ptr<float>(), x.data_ptr<float>(), yp, w.data_ptr<float>(),
                    mu.data_ptr<float>(), state.data_ptr<float>(), row_seq.data_ptr<int>(), positions.data_ptr<int64_t>(),
                    start_pos.data_ptr<int>(), slots.data_ptr<int>(), T, W, (int)groups, (int)n_mix, (float)eps,
                    is_bf(out), y_bf, store_state, cur());
}

void shift_state_update(torch::Tensor x, torch::Tensor w, double eps, torch::Tensor state, torch::Tensor cu_q,
                        torch::Tensor slots, int64_t groups) {
  chk_f32(x, "x");
  TORCH_CHECK(x.dim() == 2, "shift_state_update: x [T, W]");
  const int64_t W = x.size(1), S = slots.numel();
  chk_f32(w, "w", W); chk_f32(state, "state");
  TORCH_CHECK(state.dim() == 2 && state.size(1) == W, "shift_state_update: state must be [slots, W]");
  chk_i32(cu_q, "cu_q", S + 1); chk_i32(slots, "slots");
  TORCH_CHECK(groups >= 1 && W % groups == 0, "shift_state_update: the width must split into the norm groups");
  launch_shift_state(x.data_ptr<float>(), w.data_ptr<float>(), state.data_ptr<float>(), cu_q.data_ptr<int>(),
                     slots.data_ptr<int>(), S, W, (int)groups, (float)eps, cur());
}

void qk_prep(torch::Tensor q, torch::Tensor proj, int64_t q_off, int64_t k_off, int64_t v_off, bool v_from_k,
             c10::optional<torch::Tensor> inv_freq, double eps, torch::Tensor positions, torch::Tensor kc,
             torch::Tensor vc, torch::Tensor slot_mapping, int64_t layout, c10::optional<torch::Tensor> q_scale,
             c10::optional<torch::Tensor> q_w, c10::optional<torch::Tensor> k_w, bool v_norm, double qt_coef,
             int64_t qt_every) {
  chk_act(q, "q"); chk_act(proj, "proj"); chk_act(kc, "k_cache"); chk_act(vc, "v_cache");
  TORCH_CHECK(q.scalar_type() == proj.scalar_type() && kc.scalar_type() == proj.scalar_type() &&
              vc.scalar_type() == proj.scalar_type(), "qk_prep: one dtype for proj, q and the cache");
  TORCH_CHECK(q.dim() == 3 && proj.dim() == 2 && kc.dim() == 4 && vc.dim() == 4, "qk_prep: ranks");
  const int64_t T = q.size(0), H = q.size(1), Dk = q.size(2);
  TORCH_CHECK(layout == 0 || layout == 1, "qk_prep: layout 0 (rows) or 1 (matrix-core kernels)");
  // layout 1: values transposed per block, [nb, G, Dv, BS]; keys chunk-major in 32-entry chunks
  const int64_t G = kc.size(1), BS = kc.size(2), Dv = vc.size(layout ? 2 : 3), N = proj.size(1);
  TORCH_CHECK(proj.size(0) == T && kc.size(3) == Dk && vc.size(0) == kc.size(0) && vc.size(1) == G &&
              vc.size(layout ? 3 : 2) == BS, "qk_prep: shapes");
  TORCH_CHECK(layout == 0 || Dk % 32 == 0, "qk_prep: the matrix-core key layout needs dim % 32 == 0");
  const float* qs = nullptr;
  if (q_scale.has_value()) {
    chk_f32(*q_scale, "q_scale", H);
    qs = q_scale->data_ptr<float>();
  }
  TORCH_CHECK(Dk >= 1 && Dk <= 256 && Dv >= 1 && Dv <= 256, "qk_prep: head sizes must be 1..256");
  TORCH_CHECK(q_off >= 0 && q_off + H * Dk <= N && k_off >= 0 && k_off + G * Dk <= N, "qk_prep: q / k columns");
  TORCH_CHECK(v_from_k ? Dv == Dk : (v_off >= 0 && v_off + G * Dv <= N), "qk_prep: v columns");
  int64_t rot_dims = 0;
  const float* fr = nullptr;
  if (inv_freq.has_value()) {
    chk_f32(*inv_freq, "inv_freq");
    rot_dims = 2 * inv_freq->numel();
    TORCH_CHECK(rot_dims <= Dk, "qk_prep: more rotated entries than the head has");
    fr = inv_freq->data_ptr<float>();
  }
  chk_i64(positions, "positions", T); chk_i64(slot_mapping, "slot_mapping", T);
  const float *qw = nullptr, *kw = nullptr;
  if (q_w.has_value()) { chk_f32(*q_w, "q_w", Dk); qw = q_w->data_ptr<float>(); }
  if (k_w.has_value()) { chk_f32(*k_w, "k_w", Dk); kw = k_w->data_ptr<float>(); }
  TORCH_CHECK(qt_every >= 0 && qt_every < (int64_t(1) << 31), "qk_prep: q_temp every");
  launch_qk_prep(q.data_ptr(), proj.data_ptr(), N, q_off, k_off, v_off, v_from_k, fr, rot_dims, (float)eps,
                 positions.data_ptr<int64_t>(), kc.data_ptr(), vc.data_ptr(), slot_mapping.data_ptr<int64_t>(), T, H, G,
                 Dk, Dv, BS, is_bf(q), (int)layout, qs, qw, kw, v_norm, (float)qt_coef, (int)qt_every, cur());
}

void gqa_attention(torch::Tensor out, torch::Tensor q, torch::Tensor kc, torch::Tensor vc, torch::Tensor block_tables,
                   torch::Tensor cu_q, torch::Tensor start_pos, torch::Tensor tiles, c10::optional<torch::Tensor> temp,
                   double scale, double sink, int64_t rows, int64_t num_splits, c10::optional<torch::Tensor> part_o,
                   c10::optional<torch::Tensor> part_ml, int64_t window, c10::optional<torch::Tensor> slopes,
                   c10::optional<torch::Tensor> gate, int64_t gate_off, int64_t layout) {
  chk_act(out, "out"); chk_act(q, "q"); chk_act(kc, "k_cache"); chk_act(vc, "v_cache");
  TORCH_CHECK(out.scalar_type() == q.scalar_type() && kc.scalar_type() == q.scalar_type() &&
              vc.scalar_type() == q.scalar_type(), "gqa_attention: one dtype for q, the cache and out");
  TORCH_CHECK(q.dim() == 3 && kc.dim() == 4 && vc.dim() == 4 && out.dim() == 2, "gqa_attention: ranks");
  const int64_t T = q.size(0), H = q.size(1), Dk = q.size(2);
  TORCH_CHECK(layout == 0 || layout == 1, "gqa_attention: layout 0 (rows) or 1 (matrix-core kernels)");
  const int64_t G = kc.size(1), BS = kc.size(2), Dv = vc.size(layout ? 2 : 3);
  TORCH_CHECK(kc.size(3) == Dk && vc.size(0) == kc.size(0) && vc.size(1) == G && vc.size(layout ? 3 : 2) == BS &&
              H % G == 0, "gqa_attention: cache shapes");
  TORCH_CHECK(layout == 0 || Dk % 32 == 0, "gqa_attention: the matrix-core key layout needs dim % 32 == 0");
  TORCH_CHECK(out.size(0) == T && out.size(1) == H * Dv, "gqa_attention: out [T, H * Dv]");
  chk_i32(block_tables, "block_tables"); chk_i32(cu_q, "cu_q"); chk_i32(start_pos, "start_pos", cu_q.numel() - 1);
  chk_i32(tiles, "tiles");
  TORCH_CHECK(block_tables.dim() == 2 && block_tables.size(0) == start_pos.numel(), "gqa_attention: block_tables [S, n]");
  TORCH_CHECK(tiles.dim() == 2 && tiles.size(1) == 2, "gqa_attention: tiles [n, 2]");
  TORCH_CHECK(num_splits >= 1 && num_splits <= 64, "gqa_attention: num_splits must be 1..64");
  TORCH_CHECK(rows >= 1, "gqa_attention: rows per tile");
  const float* tp = nullptr;
  if (temp.has_value()) {
    chk_f32(*temp, "temp", H);
    tp = temp->data_ptr<float>();
  }
  float *po = nullptr, *pml = nullptr;
  if (num_splits > 1) {
    TORCH_CHECK(rows == 1, "gqa_attention: split keys need one row per tile");
    TORCH_CHECK(part_o.has_value() && part_ml.has_value(), "gqa_attention: split keys need the partial buffers");
    chk_f32(*part_o, "part_o"); chk_f32(*part_ml, "part_ml");
    TORCH_CHECK(part_o->numel() >= T * H * num_splits * Dv && part_ml->numel() >= T * H * num_splits * 2,
                "gqa_attention: partial buffers too small");
    po = part_o->data_ptr<float>();
    pml = part_ml->data_ptr<float>();
  }
  const float* sl = nullptr;
  if (slopes.has_value()) { chk_f32(*slopes, "slopes", H); sl = slopes->data_ptr<float>(); }
  TORCH_CHECK(window >= 0 && window < (int64_t(1) << 31), "gqa_attention: window");
  const char* gp = nullptr;
  int64_t gstride = 0;
  if (gate.has_value()) {      // columns gate_off .. gate_off + H * Dv of a [T, N] tensor
    chk_act(*gate, "gate");
    TORCH_CHECK(gate->dim() == 2 && gate->size(0) == T && gate->scalar_type() == q.scalar_type() && gate_off >= 0 &&
                gate_off + H * Dv <= gate->size(1), "gqa_attention: gate columns");
    gstride = gate->size(1);
    gp = static_cast<const char*>(gate->data_ptr()) + gate_off * gate->element_size();
  }
  int rc = launch_gqa_attention(out.data_ptr(), q.data_ptr(), kc.data_ptr(), vc.data_ptr(), block_tables.data_ptr<int>(),
                                cu_q.data_ptr<int>(), start_pos.data_ptr<int>(), tiles.data_ptr<int>(), tiles.size(0), tp,
                                po, pml, T, H, G, Dk, Dv, BS, block_tables.size(1), rows, num_splits, (float)scale,
                                (float)sink, (int)window, sl, gp, (int)gstride, (int)layout, is_bf(q), cur());
  TORCH_CHECK(rc == 0, "gqa_attention: unsupported shape (code ", rc, ": -1 head sizes beyond 256 or the LDS tile, "
              "-2 rows per tile, -3 LDS size refused)");
}

void mingru_scan(torch::Tensor out, torch::Tensor proj, int64_t z_off, int64_t x_off, int64_t g_off, torch::Tensor bz,
                 torch::Tensor bx, torch::Tensor state, torch::Tensor cu_q, torch::Tensor start_pos, torch::Tensor slots,
                 c10::optional<torch::Tensor> chunks, c10::optional<torch::Tensor> seq_chunk0,
                 c10::optional<torch::Tensor> ws) {
  chk_act(out, "out"); chk_act(proj, "proj");
  TORCH_CHECK(out.dim() == 2 && proj.dim() == 2 && out.size(0) == proj.size(0) && out.scalar_type() == proj.scalar_type(),
              "mingru_scan: shapes");
  const int64_t width = out.size(1), N = proj.size(1), S = slots.numel();
  for (int64_t off : {z_off, x_off, g_off}) TORCH_CHECK(off >= 0 && off + width <= N, "mingru_scan: columns");
  chk_f32(bz, "bz", width); chk_f32(bx, "bx", width); chk_f32(state, "state");
  TORCH_CHECK(state.dim() == 2 && state.size(1) == width, "mingru_scan: state must be [slots, width]");
  chk_i32(cu_q, "cu_q", S + 1); chk_i32(start_pos, "start_pos", S); chk_i32(slots, "slots");
  if (chunks.has_value()) {      // long spans: the three-launch chunked scan
    TORCH_CHECK(seq_chunk0.has_value() && ws.has_value(), "mingru_scan: chunks need seq_chunk0 and the workspace");
    chk_i32(*chunks, "chunks"); chk_i32(*seq_chunk0, "seq_chunk0", S + 1); chk_f32(*ws, "ws");
    TORCH_CHECK(chunks->dim() == 2 && chunks->size(1) == 2, "mingru_scan: chunks [n, 2]");
    const int64_t n = chunks->size(0);
    TORCH_CHECK(ws->numel() >= 3 * n * width, "mingru_scan: workspace too small");
    launch_mingru_chunked(out.data_ptr(), proj.data_ptr(), N, z_off, x_off, g_off, width, bz.data_ptr<float>(),
                          bx.data_ptr<float>(), state.data_ptr<float>(), cu_q.data_ptr<int>(), start_pos.data_ptr<int>(),
                          slots.data_ptr<int>(), S, chunks->data_ptr<int>(), n, seq_chunk0->data_ptr<int>(),
                          ws->data_ptr<float>(), is_bf(proj), cur());
    return;
  }
  launch_mingru_scan(out.data_ptr(), proj.data_ptr(), N, z_off, x_off, g_off, width, bz.data_ptr<float>(),
                     bx.data_ptr<float>(), state.data_ptr<float>(), cu_q.data_ptr<int>(), start_pos.data_ptr<int>(),
                     slots.data_ptr<int>(), S, is_bf(proj), cur());
}

void dual_norm_add(torch::Tensor x, torch::Tensor a, torch::Tensor wa, torch::Tensor b, torch::Tensor wb, double eps) {
  chk_f32(x, "x"); chk_act(a, "a"); chk_act(b, "b");
  TORCH_CHECK(x.dim() == 2 && a.sizes() == x.sizes() && b.sizes() == x.sizes() && a.scalar_type() == b.scalar_type(),
              "dual_norm_add: shapes");
  chk_f32(wa, "wa", x.size(1)); chk_f32(wb, "wb", x.size(1));
  launch_dual_norm_add(x.data_ptr<float>(), a.data_ptr(), wa.data_ptr<float>(), b.data_ptr(), wb.data_ptr<float>(),
                       x.size(0), x.size(1), (float)eps, is_bf(a), cur());
}

void add_norm(torch::Tensor out, torch::Tensor x, c10::optional<torch::Tensor> y, torch::Tensor w, double eps,
              int64_t groups) {
  chk_act(out, "out"); chk_f32(x, "x");
  TORCH_CHECK(x.dim() == 2 && out.sizes() == x.sizes(), "add_norm: shapes");
  TORCH_CHECK(groups >= 1 && x.size(1) % groups == 0, "add_norm: the width must split into the norm groups");
  chk_f32(w, "w", x.size(1));
  const void* yp = nullptr;
  bool y_bf = false;
  if (y.has_value()) {
    chk_act(*y, "y");
    TORCH_CHECK(y->sizes() == x.sizes(), "add_norm: y must have x's shape");
    yp = y->data_ptr();
    y_bf = is_bf(*y);
  }
  launch_add_norm(out.data_ptr(), x.data_ptr<float>(), yp, w.data_ptr<float>(), x.size(0), x.size(1), (int)groups,
                  (float)eps, is_bf(out), y_bf, cur());
}

void limited_glu(torch::Tensor out, torch::Tensor gu, double limit) {
  chk_act(out, "out"); chk_act(gu, "gu");
  TORCH_CHECK(gu.dim() == 2 && out.dim() == 2 && gu.size(1) == 2 * out.size(1) && gu.size(0) == out.size(0) &&
              out.scalar_type() == gu.scalar_type(), "limited_glu: gu [T, 2F] -> out [T, F]");
  launch_limited_glu(out.data_ptr(), gu.data_ptr(), gu.size(0), out.size(1), (float)limit, is_bf(gu), cur());
}

// rkvg [4, T, H * D] = the projected r, k, v and gate; lw [T, H * D] the decay's low-rank path
void wkv_scan(torch::Tensor out, torch::Tensor rkvg, torch::Tensor lw, torch::Tensor w0, torch::Tensor u,
              torch::Tensor norm_w, double eps, torch::Tensor state, torch::Tensor cu_q, torch::Tensor start_pos,
              torch::Tensor slots, c10::optional<torch::Tensor> chunks, c10::optional<torch::Tensor> seq_chunk0,
              c10::optional<torch::Tensor> ws) {
  chk_act(out, "out"); chk_act(rkvg, "rkvg"); chk_act(lw, "lw");
  TORCH_CHECK(rkvg.dim() == 3 && rkvg.size(0) == 4 && out.dim() == 2 && lw.dim() == 2, "wkv_scan: ranks");
  const int64_t T = rkvg.size(1), HD = rkvg.size(2), S = slots.numel();
  TORCH_CHECK(out.size(0) == T && out.size(1) == HD && lw.size(0) == T && lw.size(1) == HD &&
              out.scalar_type() == rkvg.scalar_type() && lw.scalar_type() == rkvg.scalar_type(), "wkv_scan: shapes");
  TORCH_CHECK(u.dim() == 2, "wkv_scan: u [heads, dim]");
  const int64_t H = u.size(0), D = u.size(1);
  TORCH_CHECK(H * D == HD && D >= 1 && D <= 256, "wkv_scan: heads x dim must be the projection width, dim 1..256");
  chk_f32(u, "u"); chk_f32(w0, "w0", HD); chk_f32(norm_w, "norm_w", HD); chk_f32(state, "state");
  TORCH_CHECK(state.dim() == 2 && state.size(1) == H * D * D, "wkv_scan: state must be [slots, heads * dim * dim]");
  chk_i32(cu_q, "cu_q", S + 1); chk_i32(start_pos, "start_pos", S); chk_i32(slots, "slots");
  const int* ch = nullptr;
  const int* sc0 = nullptr;
  float* wsp = nullptr;
  int64_t n = 0;
  if (chunks.has_value()) {
    TORCH_CHECK(seq_chunk0.has_value() && ws.has_value(), "wkv_scan: chunks need seq_chunk0 and the workspace");
    chk_i32(*chunks, "chunks"); chk_i32(*seq_chunk0, "seq_chunk0", S + 1); chk_f32(*ws, "ws");
    TORCH_CHECK(chunks->dim() == 2 && chunks->size(1) == 2, "wkv_scan: chunks [n, 2]");
    n = chunks->size(0);
    TORCH_CHECK(ws->numel() >= n * H * (D * D + D), "wkv_scan: workspace too small");
    ch = chunks->data_ptr<int>(); sc0 = seq_chunk0->data_ptr<int>(); wsp = ws->data_ptr<float>();
  }
  const char* base = static_cast<const char*>(rkvg.data_ptr());
  const int64_t plane = T * HD * rkvg.element_size();
  int rc = launch_wkv_scan(out.data_ptr(), base, base + plane, base + 2 * plane, base + 3 * plane, lw.data_ptr(), HD, HD,
                           w0.data_ptr<float>(), u.data_ptr<float>(), norm_w.data_ptr<float>(), state.data_ptr<float>(),
                           cu_q.data_ptr<int>(), start_pos.data_ptr<int>(), slots.data_ptr<int>(), S, H, D, (float)eps, ch,
                           n, sc0, wsp, is_bf(rkvg), cur());
  TORCH_CHECK(rc == 0, "wkv_scan: unsupported shape (code ", rc, ")");
}

void xielu(torch::Tensor out, torch::Tensor a, c10::optional<torch::Tensor> bias, double ap, double an) {
  chk_act(out, "out"); chk_act(a, "a");
  TORCH_CHECK(a.dim() == 2 && out.sizes() == a.sizes() && out.scalar_type() == a.scalar_type(), "xielu: shapes");
  const float* bp = nullptr;
  if (bias.has_value()) { chk_f32(*bias, "bias", a.size(1)); bp = bias->data_ptr<float>(); }
  launch_xielu(out.data_ptr(), a.data_ptr(), bp, a.size(0), a.size(1), (float)ap, (float)an, is_bf(a), cur());
}

void silu_glu(torch::Tensor out, torch::Tensor gu) {
  chk_act(out, "out"); chk_act(gu, "gu");
  TORCH_CHECK(gu.dim() == 2 && out.dim() == 2 && gu.size(1) == 2 * out.size(1) && gu.size(0) == out.size(0) &&
              out.scalar_type() == gu.scalar_type(), "silu_glu: gu [T, 2F] -> out [T, F]");
  launch_silu_glu(out.data_ptr(), gu.data_ptr(), gu.size(0), out.size(1), is_bf(gu), cur());
}

void topk_softmax(torch::Tensor idx, torch::Tensor wt, torch::Tensor logits) {
  chk_f32(logits, "logits");
  TORCH_CHECK(logits.dim() == 2 && idx.dim() == 2 && idx.size(0) == logits.size(0), "topk_softmax: shapes");
  chk_i32(idx, "idx"); chk_f32(wt, "wt", idx.numel());
  int rc = launch_topk_softmax(idx.data_ptr<int>(), wt.data_ptr<float>(), logits.data_ptr<float>(), logits.size(0),
                               logits.size(1), idx.size(1), cur());
  TORCH_CHECK(rc == 0, "topk_softmax: up to 512 experts and 64 per token");
}

// wgu [E, 2F, W] (gate rows, then up rows), wd [E, W, F]; idx / wt [T, top]; hid fp32 [T, top, F] scratch
void moe_rows(torch::Tensor out, torch::Tensor hid, torch::Tensor h, torch::Tensor wgu, torch::Tensor wd, torch::Tensor idx,
              torch::Tensor wt) {
  chk_act(out, "out"); chk_act(h, "h"); chk_act(wgu, "wgu"); chk_act(wd, "wd"); chk_f32(hid, "hid");
  TORCH_CHECK(h.dim() == 2 && wgu.dim() == 3 && wd.dim() == 3 && idx.dim() == 2, "moe_rows: ranks");
  const int64_t T = h.size(0), W = h.size(1), E = wgu.size(0), F = wd.size(2), top = idx.size(1);
  TORCH_CHECK(wgu.size(1) == 2 * F && wgu.size(2) == W && wd.size(0) == E && wd.size(1) == W && idx.size(0) == T &&
              out.sizes() == h.sizes(), "moe_rows: shapes");
  TORCH_CHECK(out.scalar_type() == h.scalar_type() && wgu.scalar_type() == h.scalar_type() &&
              wd.scalar_type() == h.scalar_type(), "moe_rows: one dtype");
  chk_i32(idx, "idx"); chk_f32(wt, "wt", T * top);
  TORCH_CHECK(hid.numel() >= T * top * F, "moe_rows: scratch too small");
  int rc = launch_moe_rows(out.data_ptr(), hid.data_ptr<float>(), h.data_ptr(), wgu.data_ptr(), wd.data_ptr(),
                           idx.data_ptr<int>(), wt.data_ptr<float>(), T, W, F, top, is_bf(h), cur());
  TORCH_CHECK(rc == 0, "moe_rows: a row does not fit the LDS");
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.def("shift_norm", &shift_norm, py::arg("out"), py::arg("xs"), py::arg("x"), py::arg("y"), py::arg("w"), py::arg("eps"),
        py::arg("mu"), py::arg("state"), py::arg("row_seq"), py::arg("positions"), py::arg("start_pos"), py::arg("slots"),
        py::arg("store_state"), py::arg("groups") = 1);
  m.def("shift_state_update", &shift_state_update, py::arg("x"), py::arg("w"), py::arg("eps"), py::arg("state"),
        py::arg("cu_q"), py::arg("slots"), py::arg("groups") = 1);
  m.def("qk_prep", &qk_prep, py::arg("q"), py::arg("proj"), py::arg("q_off"), py::arg("k_off"), py::arg("v_off"),
        py::arg("v_from_k"), py::arg("inv_freq"), py::arg("eps"), py::arg("positions"), py::arg("kc"), py::arg("vc"),
        py::arg("slot_mapping"), py::arg("layout"), py::arg("q_scale"), py::arg("q_w") = py::none(),
        py::arg("k_w") = py::none(), py::arg("v_norm") = false, py::arg("qt_coef") = 0.0, py::arg("qt_every") = 0);
  m.def("gqa_key_tile", [](int64_t Dk, int64_t Dv) { return gqa_key_tile((int)Dk, (int)Dv); });
  m.def("gqa_attention", &gqa_attention, py::arg("out"), py::arg("q"), py::arg("kc"), py::arg("vc"),
        py::arg("block_tables"), py::arg("cu_q"), py::arg("start_pos"), py::arg("tiles"), py::arg("temp"), py::arg("scale"),
        py::arg("sink"), py::arg("rows"), py::arg("num_splits"), py::arg("part_o"), py::arg("part_ml"),
        py::arg("window") = 0, py::arg("slopes") = py::none(), py::arg("gate") = py::none(), py::arg("gate_off") = 0,
        py::arg("layout") = 0);
  m.def("mingru_scan", &mingru_scan, py::arg("out"), py::arg("proj"), py::arg("z_off"), py::arg("x_off"), py::arg("g_off"),
        py::arg("bz"), py::arg("bx"), py::arg("state"), py::arg("cu_q"), py::arg("start_pos"), py::arg("slots"),
        py::arg("chunks") = py::none(), py::arg("seq_chunk0") = py::none(), py::arg("ws") = py::none());
  m.def("mingru_scan_chunk", &mingru_scan_chunk);
  m.def("dual_norm_add", &dual_norm_add);
  m.def("add_norm", &add_norm, py::arg("out"), py::arg("x"), py::arg("y"), py::arg("w"), py::arg("eps"),
        py::arg("groups") = 1);
  m.def("wkv_scan", &wkv_scan, py::arg("out"), py::arg("rkvg"), py::arg("lw"), py::arg("w0"), py::arg("u"),
        py::arg("norm_w"), py::arg("eps"), py::arg("state"), py::arg("cu_q"), py::arg("start_pos"), py::arg("slots"),
        py::arg("chunks") = py::none(), py::arg("seq_chunk0") = py::none(), py::arg("ws") = py::none());
  m.def("wkv_scan_chunk", &wkv_scan_chunk);
  m.def("xielu", &xielu);
  m.def("silu_glu", &silu_glu);
  m.def("topk_softmax", &topk_softmax);
  m.def("moe_rows", &moe_rows);
  m.def("limited_glu", &limited_glu);
}
