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
                         const void* gate, int gate_stride, int layout, float softcap, float out_scale, int out_stride,
                         int out_off, bool bf, hipStream_t stream);
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
                    const float* wt, int T, int W, int F, int top, int act, bool bf, hipStream_t stream);
int launch_route_topk(int* idx, float* wt, const void* h, const float* wr, const float* bias, int T, int W, int E,
                      int top, bool bf, hipStream_t stream);
void launch_canon_add(void* h, float* xs, const float* x, const void* y, const void* y2, const float* nw, float eps,
                      const float* cw, float* state, int sub, int nsub, const int* row_seq, const int64_t* positions,
                      const int* start_pos, const int* slots, int T, int W, int taps, int keep, bool out_bf, bool y_bf,
                      bool shift_state, hipStream_t stream);
void launch_conv_state(const void* x, int stride, int col_off, int C, float* state, int sub, int nsub, int keep,
                       const int* cu_q, const int* start_pos, const int* slots, int S, bool bf, hipStream_t stream);
int launch_qkv_prep_wide(void* q, const void* proj, int stride, int q_off, int k_off, int v_off, bool v_from_k,
                         const float* qb, const float* kb, const float* qw, const float* kw, const float* freq, int R,
                         float mag, const float* vfreq, float eps, const int64_t* positions, void* kc, void* vc,
                         const int64_t* slot_mapping, int T, int H, int G, int Dk, int Dv, int BS, bool bf,
                         hipStream_t stream);
void launch_turn_back(void* out, int out_stride, int out_off, const void* o, int T, int H, int E,
                      const int64_t* positions, const float* vfreq, float scale, bool bf, hipStream_t stream);
void launch_silu_cols(float* out, const void* proj, int stride, int off, int n, int T, bool bf, hipStream_t stream);
void launch_relu2(void* out, const void* a, int64_t total, bool bf, hipStream_t stream);
void launch_removal_prep(float* out, const void* proj, int stride, int r_off, int k_off, int v_off, int a_off,
                         const void* lw, const float* w0, const float* ab, int T, int A, int D, bool bf,
                         hipStream_t stream);
int launch_delta_prep(float* five, float* vout, const void* proj, int stride, int q_off, int b_off, int a_off,
                      const float* cw, float* state, const float* neg_rate, const float* dt_bias, int T, int A, int G,
                      int D, int E, int taps, int keep, const int* row_seq, const int64_t* positions,
                      const int* start_pos, const int* slots, bool shift_state, bool bf, hipStream_t stream);
void launch_head_norm_gate(void* out, int out_stride, int out_off, const float* o, const float* w, int wmod, int span,
                           const void* gate, int gate_stride, int gate_off, int act, float eps, float scale, int T, int C,
                           bool out_bf, bool gate_bf, hipStream_t stream);
int launch_state_scan(float* out, const float* q, const float* k, const float* v, const float* w, const float* a,
                      const float* b, int sq, int sk, int sv, int sw, int sa, int sb, const float* decay, float* state,
                      const int* cu_q, const int* start_pos, const int* slots, int S, int T, int A, int D, int E,
                      hipStream_t stream);

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
                   c10::optional<torch::Tensor> gate, int64_t gate_off, int64_t layout, double softcap, double out_scale,
                   int64_t out_off) {
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
  TORCH_CHECK(out.size(0) == T && out_off >= 0 && out_off + H * Dv <= out.size(1) && softcap >= 0,
              "gqa_attention: out [T, >= out_off + H * Dv]");
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
                                (float)sink, (int)window, sl, gp, (int)gstride, (int)layout, (float)softcap,
                                (float)out_scale, (int)out.size(1), (int)out_off, is_bf(q), cur());
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
void route_topk(torch::Tensor idx, torch::Tensor wt, torch::Tensor h, torch::Tensor wr, c10::optional<torch::Tensor> bias) {
  chk_act(h, "h"); chk_f32(wr, "router"); chk_i32(idx, "idx"); chk_f32(wt, "wt", idx.numel());
  TORCH_CHECK(h.dim() == 2 && wr.dim() == 2 && idx.dim() == 2 && wr.size(1) == h.size(1) && idx.size(0) == h.size(0),
              "route_topk: h [T, W], router [E, W], idx [T, top]");
  const float* bp = nullptr;
  if (bias.has_value()) { chk_f32(*bias, "bias", wr.size(0)); bp = bias->data_ptr<float>(); }
  int rc = launch_route_topk(idx.data_ptr<int>(), wt.data_ptr<float>(), h.data_ptr(), wr.data_ptr<float>(), bp,
                             (int)h.size(0), (int)h.size(1), (int)wr.size(0), (int)idx.size(1), is_bf(h), cur());
  TORCH_CHECK(rc == 0, "route_topk: at most 512 experts, 64 choices and a row of 48 KiB (code ", rc, ")");
}

void moe_rows(torch::Tensor out, torch::Tensor hid, torch::Tensor h, torch::Tensor wgu, torch::Tensor wd, torch::Tensor idx,
              torch::Tensor wt, int64_t act) {
  chk_act(out, "out"); chk_act(h, "h"); chk_act(wgu, "wgu"); chk_act(wd, "wd"); chk_f32(hid, "hid");
  TORCH_CHECK(h.dim() == 2 && wgu.dim() == 3 && wd.dim() == 3 && idx.dim() == 2, "moe_rows: ranks");
  const int64_t T = h.size(0), W = h.size(1), E = wgu.size(0), F = wd.size(2), top = idx.size(1);
  TORCH_CHECK((act == 0 || act == 1) && wgu.size(1) == (act ? 1 : 2) * F && wgu.size(2) == W && wd.size(0) == E && wd.size(1) == W && idx.size(0) == T &&
              out.sizes() == h.sizes(), "moe_rows: shapes");
  TORCH_CHECK(out.scalar_type() == h.scalar_type() && wgu.scalar_type() == h.scalar_type() &&
              wd.scalar_type() == h.scalar_type(), "moe_rows: one dtype");
  chk_i32(idx, "idx"); chk_f32(wt, "wt", T * top);
  TORCH_CHECK(hid.numel() >= T * top * F, "moe_rows: scratch too small");
  int rc = launch_moe_rows(out.data_ptr(), hid.data_ptr<float>(), h.data_ptr(), wgu.data_ptr(), wd.data_ptr(),
                           idx.data_ptr<int>(), wt.data_ptr<float>(), T, W, F, top, (int)act, is_bf(h), cur());
  TORCH_CHECK(rc == 0, "moe_rows: a row does not fit the LDS");
}

using OptT = c10::optional<torch::Tensor>;

const float* opt_f32(const OptT& t, const char* name, int64_t n) {
  if (!t.has_value()) return nullptr;
  chk_f32(*t, name, n);
  return t->data_ptr<float>();
}

// rows [T] / spans [S] of a batch, checked against each other
void chk_rows(const torch::Tensor& row_seq, const torch::Tensor& positions, const torch::Tensor& start_pos,
              const torch::Tensor& slots, int64_t T, int64_t n_slots) {
  chk_i32(row_seq, "row_seq", T);
  chk_i64(positions, "positions", T);
  chk_i32(start_pos, "start_pos");
  chk_i32(slots, "slots", start_pos.numel());
  (void)n_slots;
}

void canon_add(OptT h, torch::Tensor xs, torch::Tensor x, OptT y, OptT y2, OptT nw, double eps, OptT cw, OptT state,
               int64_t sub, torch::Tensor row_seq, torch::Tensor positions, torch::Tensor start_pos, torch::Tensor slots,
               bool shift_state) {
  chk_f32(x, "x"); chk_f32(xs, "xs", x.numel());
  TORCH_CHECK(x.dim() == 2, "canon_add: x [T, W]");
  const int64_t T = x.size(0), W = x.size(1);
  if (T == 0 || (!y.has_value() && !cw.has_value())) return;
  bool y_bf = false;
  if (y.has_value()) {
    chk_act(*y, "y");
    TORCH_CHECK(y->numel() == x.numel() && nw.has_value() && xs.data_ptr() != x.data_ptr(),
                "canon_add: y [T, W] needs the norm weight and an output of its own");
    y_bf = is_bf(*y);
    if (y2.has_value()) {
      chk_act(*y2, "y2");
      TORCH_CHECK(y2->numel() == x.numel() && y2->scalar_type() == y->scalar_type(), "canon_add: y2 like y");
    }
  } else {
    TORCH_CHECK(xs.data_ptr() == x.data_ptr() && !y2.has_value(), "canon_add: without y the residual is x itself");
  }
  int taps = 0, keep = 0, nsub = 1;
  void* hp = nullptr;
  bool out_bf = false;
  if (cw.has_value()) {
    chk_f32(*cw, "conv_w");
    TORCH_CHECK(cw->dim() == 2 && cw->size(0) == W && cw->size(1) >= 1 && cw->size(1) <= 16, "canon_add: conv_w [W, taps <= 16]");
    taps = (int)cw->size(1);
    TORCH_CHECK(h.has_value() && state.has_value(), "canon_add: the convolution needs h and the state");
    chk_act(*h, "h");
    TORCH_CHECK(h->numel() == x.numel(), "canon_add: h [T, W]");
    chk_f32(*state, "state");
    TORCH_CHECK(state->dim() == 4 && state->size(3) == W && state->size(2) >= std::max(taps - 1, 1) && sub >= 0 &&
                sub < state->size(1), "canon_add: state [slots, subs, taps - 1, W]");
    TORCH_CHECK(state->size(2) == std::max(taps - 1, 1), "canon_add: state rows");
    keep = (int)state->size(2);
    nsub = (int)state->size(1);
    chk_rows(row_seq, positions, start_pos, slots, T, state->size(0));
    hp = h->data_ptr();
    out_bf = is_bf(*h);
  }
  launch_canon_add(hp, xs.data_ptr<float>(), x.data_ptr<float>(), y.has_value() ? y->data_ptr() : nullptr,
                   y2.has_value() ? y2->data_ptr() : nullptr, opt_f32(nw, "norm_w", W), (float)eps,
                   cw.has_value() ? cw->data_ptr<float>() : nullptr, cw.has_value() ? state->data_ptr<float>() : nullptr,
                   (int)sub, nsub, cw.has_value() ? row_seq.data_ptr<int>() : nullptr,
                   cw.has_value() ? positions.data_ptr<int64_t>() : nullptr,
                   cw.has_value() ? start_pos.data_ptr<int>() : nullptr, cw.has_value() ? slots.data_ptr<int>() : nullptr,
                   (int)T, (int)W, taps, keep, out_bf, y_bf, shift_state, cur());
}

void conv_state_update(torch::Tensor x, int64_t col_off, int64_t C, torch::Tensor state, int64_t sub, torch::Tensor cu_q,
                       torch::Tensor start_pos, torch::Tensor slots) {
  chk_act(x, "x"); chk_f32(state, "state");
  TORCH_CHECK(x.dim() == 2 && col_off >= 0 && col_off + C <= x.size(1), "conv_state_update: columns");
  TORCH_CHECK((state.dim() == 4 || state.dim() == 3) && state.size(-1) == C && state.size(-2) <= 16,
              "conv_state_update: state [slots, (subs,) keep, C]");
  const int nsub = state.dim() == 4 ? (int)state.size(1) : 1;
  TORCH_CHECK(sub >= 0 && sub < nsub, "conv_state_update: sub");
  const int64_t S = cu_q.numel() - 1;
  chk_i32(cu_q, "cu_q"); chk_i32(start_pos, "start_pos", S); chk_i32(slots, "slots", S);
  launch_conv_state(x.data_ptr(), (int)x.size(1), (int)col_off, (int)C, state.data_ptr<float>(), (int)sub, nsub,
                    (int)state.size(-2), cu_q.data_ptr<int>(), start_pos.data_ptr<int>(), slots.data_ptr<int>(), (int)S,
                    is_bf(x), cur());
}

void qkv_prep_wide(torch::Tensor q, torch::Tensor proj, int64_t q_off, int64_t k_off, int64_t v_off, bool v_from_k,
                   OptT qb, OptT kb, torch::Tensor qw, torch::Tensor kw, OptT freq, double mag, OptT vfreq, double eps,
                   torch::Tensor positions, torch::Tensor kc, torch::Tensor vc, torch::Tensor slot_mapping) {
  chk_act(q, "q"); chk_act(proj, "proj"); chk_act(kc, "k_cache"); chk_act(vc, "v_cache");
  TORCH_CHECK(q.dim() == 3 && proj.dim() == 2 && kc.dim() == 4 && vc.dim() == 4, "qkv_prep_wide: ranks");
  TORCH_CHECK(q.scalar_type() == proj.scalar_type() && kc.scalar_type() == proj.scalar_type() &&
              vc.scalar_type() == proj.scalar_type(), "qkv_prep_wide: one dtype");
  const int64_t T = q.size(0), H = q.size(1), Dk = q.size(2), G = kc.size(1), BS = kc.size(2), Dv = vc.size(3), N = proj.size(1);
  TORCH_CHECK(proj.size(0) == T && kc.size(3) == Dk && vc.size(0) == kc.size(0) && vc.size(1) == G && vc.size(2) == BS,
              "qkv_prep_wide: shapes");
  TORCH_CHECK(q_off >= 0 && q_off + H * Dk <= N && k_off >= 0 && k_off + G * Dk <= N, "qkv_prep_wide: q / k columns");
  TORCH_CHECK(v_from_k ? Dv == Dk : (v_off >= 0 && v_off + G * Dv <= N), "qkv_prep_wide: value columns");
  chk_f32(qw, "q_w", H * Dk); chk_f32(kw, "k_w", G * Dk);
  int R = 0;
  if (freq.has_value()) {
    chk_f32(*freq, "freq");
    R = (int)freq->numel();
    TORCH_CHECK(2 * R <= Dk, "qkv_prep_wide: rotated entries beyond the head");
  }
  if (vfreq.has_value()) {
    chk_f32(*vfreq, "vfreq", Dv / 2);
    TORCH_CHECK(Dv % 2 == 0 && !v_from_k, "qkv_prep_wide: turned values need an even vdim and a value projection");
  }
  chk_i64(positions, "positions", T); chk_i64(slot_mapping, "slot_mapping", T);
  int rc = launch_qkv_prep_wide(q.data_ptr(), proj.data_ptr(), (int)N, (int)q_off, (int)k_off, (int)v_off, v_from_k,
                                opt_f32(qb, "q_bias", H * Dk), opt_f32(kb, "k_bias", G * Dk), qw.data_ptr<float>(),
                                kw.data_ptr<float>(), freq.has_value() ? freq->data_ptr<float>() : nullptr, R, (float)mag,
                                vfreq.has_value() ? vfreq->data_ptr<float>() : nullptr, (float)eps,
                                positions.data_ptr<int64_t>(), kc.data_ptr(), vc.data_ptr(),
                                slot_mapping.data_ptr<int64_t>(), (int)T, (int)H, (int)G, (int)Dk, (int)Dv, (int)BS,
                                is_bf(proj), cur());
  TORCH_CHECK(rc == 0, "qkv_prep_wide: the query and key rows do not fit the LDS (code ", rc, ")");
}

void turn_back(torch::Tensor out, int64_t out_off, torch::Tensor o, int64_t H, torch::Tensor positions,
               torch::Tensor vfreq, double scale) {
  chk_act(out, "out"); chk_act(o, "o");
  TORCH_CHECK(out.dim() == 2 && o.dim() == 2 && out.size(0) == o.size(0) && out.scalar_type() == o.scalar_type() &&
              H >= 1 && o.size(1) % H == 0 && out_off >= 0 && out_off + o.size(1) <= out.size(1), "turn_back: shapes");
  const int64_t E = o.size(1) / H;
  TORCH_CHECK(E % 2 == 0, "turn_back: even head size");
  chk_f32(vfreq, "vfreq", E / 2); chk_i64(positions, "positions", o.size(0));
  launch_turn_back(out.data_ptr(), (int)out.size(1), (int)out_off, o.data_ptr(), (int)o.size(0), (int)H, (int)E,
                   positions.data_ptr<int64_t>(), vfreq.data_ptr<float>(), (float)scale, is_bf(o), cur());
}

void silu_cols(torch::Tensor out, torch::Tensor proj, int64_t off) {
  chk_f32(out, "out"); chk_act(proj, "proj");
  TORCH_CHECK(out.dim() == 2 && proj.dim() == 2 && out.size(0) == proj.size(0) && off >= 0 &&
              off + out.size(1) <= proj.size(1), "silu_cols: columns");
  launch_silu_cols(out.data_ptr<float>(), proj.data_ptr(), (int)proj.size(1), (int)off, (int)out.size(1),
                   (int)out.size(0), is_bf(proj), cur());
}

void relu2(torch::Tensor out, torch::Tensor a) {
  chk_act(out, "out"); chk_act(a, "a");
  TORCH_CHECK(out.numel() == a.numel() && out.scalar_type() == a.scalar_type(), "relu2: out like a");
  launch_relu2(out.data_ptr(), a.data_ptr(), a.numel(), is_bf(a), cur());
}

void removal_prep(torch::Tensor out, torch::Tensor proj, int64_t r_off, int64_t k_off, int64_t v_off, int64_t a_off,
                  torch::Tensor lw, torch::Tensor w0, torch::Tensor ab, int64_t A) {
  chk_f32(out, "out"); chk_act(proj, "proj"); chk_act(lw, "lw");
  TORCH_CHECK(out.dim() == 3 && out.size(0) == 6 && proj.dim() == 2 && out.size(1) == proj.size(0) && A >= 1 &&
              out.size(2) % A == 0, "removal_prep: out [6, T, A * D]");
  const int64_t T = proj.size(0), n = out.size(2), N = proj.size(1);
  for (int64_t o : {r_off, k_off, v_off, a_off}) TORCH_CHECK(o >= 0 && o + n <= N, "removal_prep: columns");
  TORCH_CHECK(lw.dim() == 2 && lw.size(0) == T && lw.size(1) == n && lw.scalar_type() == proj.scalar_type(),
              "removal_prep: lw [T, A * D] of proj's dtype");
  chk_f32(w0, "w0", n); chk_f32(ab, "a_bias", n);
  launch_removal_prep(out.data_ptr<float>(), proj.data_ptr(), (int)N, (int)r_off, (int)k_off, (int)v_off, (int)a_off,
                      lw.data_ptr(), w0.data_ptr<float>(), ab.data_ptr<float>(), (int)T, (int)A, (int)(n / A),
                      is_bf(proj), cur());
}

void delta_prep(torch::Tensor five, torch::Tensor vout, torch::Tensor proj, int64_t q_off, int64_t b_off, int64_t a_off,
                torch::Tensor cw, torch::Tensor state, torch::Tensor neg_rate, torch::Tensor dt_bias, int64_t A, int64_t G,
                int64_t D, int64_t E, torch::Tensor row_seq, torch::Tensor positions, torch::Tensor start_pos,
                torch::Tensor slots, bool shift_state) {
  chk_act(proj, "proj");
  TORCH_CHECK(proj.dim() == 2 && A >= 1 && G >= 1 && A % G == 0 && D >= 1 && E >= 1, "delta_prep: sizes");
  const int64_t T = proj.size(0), N = proj.size(1), C = 2 * G * D + A * E;
  chk_f32(five, "five", 5 * T * A * D); chk_f32(vout, "v", T * A * E);
  TORCH_CHECK(q_off >= 0 && q_off + C <= N && b_off >= 0 && b_off + A <= N && a_off >= 0 && a_off + A <= N,
              "delta_prep: columns");
  chk_f32(cw, "conv_w");
  TORCH_CHECK(cw.dim() == 2 && cw.size(0) == C && cw.size(1) >= 1 && cw.size(1) <= 16, "delta_prep: conv_w [C, taps <= 16]");
  const int taps = (int)cw.size(1);
  chk_f32(state, "state");
  TORCH_CHECK(state.dim() == 3 && state.size(2) == C && state.size(1) == std::max(taps - 1, 1),
              "delta_prep: state [slots, taps - 1, C]");
  chk_f32(neg_rate, "neg_rate", A); chk_f32(dt_bias, "dt_bias", A);
  chk_rows(row_seq, positions, start_pos, slots, T, state.size(0));
  int rc = launch_delta_prep(five.data_ptr<float>(), vout.data_ptr<float>(), proj.data_ptr(), (int)N, (int)q_off,
                             (int)b_off, (int)a_off, cw.data_ptr<float>(), state.data_ptr<float>(),
                             neg_rate.data_ptr<float>(), dt_bias.data_ptr<float>(), (int)T, (int)A, (int)G, (int)D, (int)E,
                             taps, (int)state.size(1), row_seq.data_ptr<int>(), positions.data_ptr<int64_t>(),
                             start_pos.data_ptr<int>(), slots.data_ptr<int>(), shift_state, is_bf(proj), cur());
  TORCH_CHECK(rc == 0, "delta_prep: a row does not fit the LDS (code ", rc, ")");
}

// an fp32 row stream [T, >= A * n] with unit column stride: pointer and row stride
const float* stream_of(const OptT& t, const char* name, int64_t T, int64_t n, int& stride) {
  stride = 0;
  if (!t.has_value()) return nullptr;
  TORCH_CHECK(t->is_cuda() && t->scalar_type() == torch::kFloat32 && t->dim() == 2 && t->size(0) == T &&
              t->size(1) == n && (t->size(1) == 1 || t->stride(1) == 1) && t->stride(0) >= n, name,
              " must be an fp32 [T, heads * size] GPU tensor with unit column stride");
  stride = (int)t->stride(0);
  return t->data_ptr<float>();
}

void state_scan(torch::Tensor out, torch::Tensor q, torch::Tensor k, torch::Tensor v, OptT w, OptT a, OptT b, OptT decay,
                torch::Tensor state, torch::Tensor cu_q, torch::Tensor start_pos, torch::Tensor slots, int64_t A, int64_t D,
                int64_t E) {
  TORCH_CHECK(A >= 1 && D >= 1 && D <= 256 && E >= 1, "state_scan: heads, dim <= 256, vdim");
  TORCH_CHECK(q.dim() == 2, "state_scan: q [T, A * D]");
  const int64_t T = q.size(0), S = cu_q.numel() - 1;
  chk_f32(out, "out", T * A * E);
  int sq, sk, sv, sw, sa, sb;
  const float* qp = stream_of(q, "q", T, A * D, sq);
  const float* kp = stream_of(k, "k", T, A * D, sk);
  const float* vp = stream_of(v, "v", T, A * E, sv);
  const float* wp = stream_of(w, "w", T, A * D, sw);
  const float* ap = stream_of(a, "a", T, A * D, sa);
  const float* bp = stream_of(b, "b", T, A * D, sb);
  TORCH_CHECK(a.has_value() == b.has_value(), "state_scan: a and b come together");
  TORCH_CHECK(w.has_value() != decay.has_value(), "state_scan: either a decay stream or a constant per head");
  chk_f32(state, "state");
  TORCH_CHECK(state.dim() == 2 && state.size(1) == A * D * E, "state_scan: state [slots, A * E * D]");
  chk_i32(cu_q, "cu_q"); chk_i32(start_pos, "start_pos", S); chk_i32(slots, "slots", S);
  int rc = launch_state_scan(out.data_ptr<float>(), qp, kp, vp, wp, ap, bp, sq, sk, sv, sw, sa, sb,
                             opt_f32(decay, "decay", A), state.data_ptr<float>(), cu_q.data_ptr<int>(),
                             start_pos.data_ptr<int>(), slots.data_ptr<int>(), (int)S, (int)T, (int)A, (int)D, (int)E, cur());
  TORCH_CHECK(rc == 0, "state_scan: unsupported shape (code ", rc, ")");
}

void head_norm_gate(torch::Tensor out, int64_t out_off, torch::Tensor o, torch::Tensor w, int64_t span, torch::Tensor gate,
                    int64_t gate_off, int64_t act, double eps, double scale) {
  chk_act(out, "out"); chk_f32(o, "o"); chk_act(gate, "gate"); chk_f32(w, "norm_w");
  TORCH_CHECK(out.dim() == 2 && o.dim() == 2 && gate.dim() == 2 && out.size(0) == o.size(0) && gate.size(0) == o.size(0),
              "head_norm_gate: ranks");
  const int64_t T = o.size(0), C = o.size(1);
  TORCH_CHECK(span >= 1 && C % span == 0 && (w.numel() == C || w.numel() == span), "head_norm_gate: span / weight");
  TORCH_CHECK(out_off >= 0 && out_off + C <= out.size(1) && gate_off >= 0 && gate_off + C <= gate.size(1),
              "head_norm_gate: columns");
  launch_head_norm_gate(out.data_ptr(), (int)out.size(1), (int)out_off, o.data_ptr<float>(), w.data_ptr<float>(),
                        (int)w.numel(), (int)span, gate.data_ptr(), (int)gate.size(1), (int)gate_off, (int)act, (float)eps,
                        (float)scale, (int)T, (int)C, is_bf(out), is_bf(gate), cur());
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
        py::arg("layout") = 0, py::arg("softcap") = 0.0, py::arg("out_scale") = 1.0, py::arg("out_off") = 0);
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
  m.def("route_topk", &route_topk);
  m.def("moe_rows", &moe_rows, py::arg("out"), py::arg("hid"), py::arg("h"), py::arg("wgu"), py::arg("wd"), py::arg("idx"),
        py::arg("wt"), py::arg("act") = 0);
  m.def("limited_glu", &limited_glu);
  m.def("canon_add", &canon_add);
  m.def("conv_state_update", &conv_state_update);
  m.def("qkv_prep_wide", &qkv_prep_wide);
  m.def("turn_back", &turn_back);
  m.def("silu_cols", &silu_cols);
  m.def("relu2", &relu2);
  m.def("removal_prep", &removal_prep);
  m.def("delta_prep", &delta_prep);
  m.def("state_scan", &state_scan);
  m.def("head_norm_gate", &head_norm_gate);
}
