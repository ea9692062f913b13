// pybind11 bindings of the grouped-attention + recurrence family (module theroundtaible_amd._C_hybrid):
// torch tensors -> raw HIP launchers on the current HIP stream, so every kernel can be captured by
// a hipGraph like any torch op. Every entry point validates dtype / device / contiguity / shape
// BEFORE launching: a hand-written kernel never sees operands its grid does not assume.
#include <torch/extension.h>
#include <c10/hip/HIPStream.h>
#include <hip/hip_runtime.h>

void launch_shift_norm(void* out, float* xs, const float* x, const void* y, const float* w, const float* mu,
                       float* state, const int* row_seq, const int64_t* positions, const int* start_pos,
                       const int* slots, int T, int W, float eps, bool out_bf, bool y_bf, bool store_state,
                       hipStream_t stream);
void launch_shift_state(const float* x, const float* w, float* state, const int* cu_q, const int* slots, int S, int W,
                        float eps, hipStream_t stream);
void launch_qk_prep(void* q, const void* proj, int stride, int q_off, int k_off, int v_off, bool v_from_k,
                    const float* inv_freq, int rot_dims, float eps, const int64_t* positions, void* kc, void* vc,
                    const int64_t* slot_mapping, int T, int H, int G, int Dk, int Dv, int BS, bool bf, int layout,
                    const float* q_scale, hipStream_t stream);
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
void launch_add_norm(void* out, float* x, const void* y, const float* w, int T, int W, float eps, bool out_bf,
                     bool y_bf, hipStream_t stream);
void launch_limited_glu(void* out, const void* gu, int64_t rows, int F, float limit, bool bf, hipStream_t stream);
int gqa_key_tile(int Dk, int Dv);
int launch_gqa_attention(void* out, const void* q, const void* kc, const void* vc, const int* block_tables,
                         const int* cu_q, const int* start_pos, const int* tiles, int n_tiles, const float* temp,
                         float* part_o, float* part_ml, int T, int H, int G, int Dk, int Dv, int BS, int max_blocks,
                         int rows, int num_splits, float scale, float sink, bool bf, hipStream_t stream);

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
                torch::Tensor start_pos, torch::Tensor slots, bool store_state) {
  chk_act(out, "out"); chk_f32(xs, "xs"); chk_f32(x, "x");
  TORCH_CHECK(x.dim() == 2 && out.sizes() == x.sizes() && xs.sizes() == x.sizes(), "shift_norm: shapes");
  const int64_t T = x.size(0), W = x.size(1);
  chk_f32(w, "w", W); chk_f32(mu, "mu", W); chk_f32(state, "state");
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
                    start_pos.data_ptr<int>(), slots.data_ptr<int>(), T, W, (float)eps, is_bf(out), y_bf, store_state,
                    cur());
}

void shift_state_update(torch::Tensor x, torch::Tensor w, double eps, torch::Tensor state, torch::Tensor cu_q,
                        torch::Tensor slots) {
  chk_f32(x, "x");
  TORCH_CHECK(x.dim() == 2, "shift_state_update: x [T, W]");
  const int64_t W = x.size(1), S = slots.numel();
  chk_f32(w, "w", W); chk_f32(state, "state");
  TORCH_CHECK(state.dim() == 2 && state.size(1) == W, "shift_state_update: state must be [slots, W]");
  chk_i32(cu_q, "cu_q", S + 1); chk_i32(slots, "slots");
  launch_shift_state(x.data_ptr<float>(), w.data_ptr<float>(), state.data_ptr<float>(), cu_q.data_ptr<int>(),
                     slots.data_ptr<int>(), S, W, (float)eps, cur());
}

void qk_prep(torch::Tensor q, torch::Tensor proj, int64_t q_off, int64_t k_off, int64_t v_off, bool v_from_k,
             c10::optional<torch::Tensor> inv_freq, double eps, torch::Tensor positions, torch::Tensor kc,
             torch::Tensor vc, torch::Tensor slot_mapping, int64_t layout, c10::optional<torch::Tensor> q_scale) {
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
  launch_qk_prep(q.data_ptr(), proj.data_ptr(), N, q_off, k_off, v_off, v_from_k, fr, rot_dims, (float)eps,
                 positions.data_ptr<int64_t>(), kc.data_ptr(), vc.data_ptr(), slot_mapping.data_ptr<int64_t>(), T, H, G,
                 Dk, Dv, BS, is_bf(q), (int)layout, qs, cur());
}

void gqa_attention(torch::Tensor out, torch::Tensor q, torch::Tensor kc, torch::Tensor vc, torch::Tensor block_tables,
                   torch::Tensor cu_q, torch::Tensor start_pos, torch::Tensor tiles, c10::optional<torch::Tensor> temp,
                   double scale, double sink, int64_t rows, int64_t num_splits, c10::optional<torch::Tensor> part_o,
                   c10::optional<torch::Tensor> part_ml) {
  chk_act(out, "out"); chk_act(q, "q"); chk_act(kc, "k_cache"); chk_act(vc, "v_cache");
  TORCH_CHECK(out.scalar_type() == q.scalar_type() && kc.scalar_type() == q.scalar_type() &&
              vc.scalar_type() == q.scalar_type(), "gqa_attention: one dtype for q, the cache and out");
  TORCH_CHECK(q.dim() == 3 && kc.dim() == 4 && vc.dim() == 4 && out.dim() == 2, "gqa_attention: ranks");
  const int64_t T = q.size(0), H = q.size(1), Dk = q.size(2);
  const int64_t G = kc.size(1), BS = kc.size(2), Dv = vc.size(3);
  TORCH_CHECK(kc.size(3) == Dk && vc.size(0) == kc.size(0) && vc.size(1) == G && vc.size(2) == BS && H % G == 0,
              "gqa_attention: cache shapes");
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
  int rc = launch_gqa_attention(out.data_ptr(), q.data_ptr(), kc.data_ptr(), vc.data_ptr(), block_tables.data_ptr<int>(),
                                cu_q.data_ptr<int>(), start_pos.data_ptr<int>(), tiles.data_ptr<int>(), tiles.size(0), tp,
                                po, pml, T, H, G, Dk, Dv, BS, block_tables.size(1), rows, num_splits, (float)scale,
                                (float)sink, is_bf(q), cur());
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

void add_norm(torch::Tensor out, torch::Tensor x, c10::optional<torch::Tensor> y, torch::Tensor w, double eps) {
  chk_act(out, "out"); chk_f32(x, "x");
  TORCH_CHECK(x.dim() == 2 && out.sizes() == x.sizes(), "add_norm: shapes");
  chk_f32(w, "w", x.size(1));
  const void* yp = nullptr;
  bool y_bf = false;
  if (y.has_value()) {
    chk_act(*y, "y");
    TORCH_CHECK(y->sizes() == x.sizes(), "add_norm: y must have x's shape");
    yp = y->data_ptr();
    y_bf = is_bf(*y);
  }
  launch_add_norm(out.data_ptr(), x.data_ptr<float>(), yp, w.data_ptr<float>(), x.size(0), x.size(1), (float)eps,
                  is_bf(out), y_bf, cur());
}

void limited_glu(torch::Tensor out, torch::Tensor gu, double limit) {
  chk_act(out, "out"); chk_act(gu, "gu");
  TORCH_CHECK(gu.dim() == 2 && out.dim() == 2 && gu.size(1) == 2 * out.size(1) && gu.size(0) == out.size(0) &&
              out.scalar_type() == gu.scalar_type(), "limited_glu: gu [T, 2F] -> out [T, F]");
  launch_limited_glu(out.data_ptr(), gu.data_ptr(), gu.size(0), out.size(1), (float)limit, is_bf(gu), cur());
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.def("shift_norm", &shift_norm);
  m.def("shift_state_update", &shift_state_update);
  m.def("qk_prep", &qk_prep);
  m.def("gqa_key_tile", [](int64_t Dk, int64_t Dv) { return gqa_key_tile((int)Dk, (int)Dv); });
  m.def("gqa_attention", &gqa_attention);
  m.def("mingru_scan", &mingru_scan, py::arg("out"), py::arg("proj"), py::arg("z_off"), py::arg("x_off"), py::arg("g_off"),
        py::arg("bz"), py::arg("bx"), py::arg("state"), py::arg("cu_q"), py::arg("start_pos"), py::arg("slots"),
        py::arg("chunks") = py::none(), py::arg("seq_chunk0") = py::none(), py::arg("ws") = py::none());
  m.def("mingru_scan_chunk", &mingru_scan_chunk);
  m.def("dual_norm_add", &dual_norm_add);
  m.def("add_norm", &add_norm);
  m.def("limited_glu", &limited_glu);
}
