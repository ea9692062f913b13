// pybind11 bindings of the latent-attention family (module theroundtaible_amd._C_latent): torch
// tensors -> raw HIP launchers on the current HIP stream, so every kernel can be captured by a
// hipGraph like any torch op. Every entry point validates dtype / device / contiguity / shape
// BEFORE launching: a hand-written kernel never sees operands its grid does not assume.
#include <torch/extension.h>
#include <c10/hip/HIPStream.h>
#include <hip/hip_runtime.h>

void launch_scalar_rms_norm(void* out, const void* x, const float* g, int rows, int W, float eps, bool in_bf,
                            bool out_bf, hipStream_t stream);
void launch_scalar_norm_add(float* res, const void* y, const float* g, int rows, int W, float eps, bool y_bf,
                            hipStream_t stream);
void launch_canon_norm(void* out, const float* x, const float* g, float eps, const float* w, float* conv, int sub,
                       const int* row_seq, const int64_t* positions, const int* start_pos, const int* slots, int T,
                       int W, int taps, int keep, bool out_bf, bool shift_state, hipStream_t stream);
void launch_canon_state(const float* x, const float* g, float eps, float* conv, int sub, const int* cu_q,
                        const int* start_pos, const int* slots, int S, int W, int taps, int keep, hipStream_t stream);
void launch_latent_prep(void* cq, const void* proj, int proj_stride, int T, int q_rank, int kv_rank, int rot_dim,
                        const float* wq, const float* wkv, float eps, const int64_t* positions, float rot_base,
                        int rot_dims, void* cache, const int64_t* slot_mapping, bool bf, hipStream_t stream);
void launch_gate_mul(void* out, const void* o, const void* proj, int proj_stride, int g_off, int T, int H, int Dv,
                     bool bf, hipStream_t stream);
void launch_poly_norm(void* out, const void* z, const float* coef, int rows, int F, float eps, bool bf,
                      hipStream_t stream);
void launch_softcap(float* out, const void* x, int64_t n, float scale, float cap, bool bf, hipStream_t stream);
int latent_rows_per_tile(int H, int C, int R, bool bf);
int launch_latent_attention(void* out, const void* q_lat, const void* q, const void* cache, const int* block_tables,
                            const int* cu_q, const int* start_pos, const int* tiles, int n_tiles, const float* sink,
                            float* part_o, float* part_ml, int T, int H, int C, int R, int Dq, int rot_off, int BS,
                            int max_blocks, int rows, int num_splits, float scale, float rot_base, int rot_dims,
                            bool bf, hipStream_t stream);

namespace {

hipStream_t cur() { return c10::hip::getCurrentHIPStream().stream(); }

bool is_bf(const torch::Tensor& t) { return t.scalar_type() == torch::kBFloat16; }

void chk(const torch::Tensor& t, const char* name, bool contiguous = true) {
  TORCH_CHECK(t.is_cuda(), name, " must be a GPU tensor");
  TORCH_CHECK(!contiguous || t.is_contiguous(), name, " must be contiguous");
}
void chk_act(const torch::Tensor& t, const char* name) {
  chk(t, name);
  TORCH_CHECK(is_bf(t) || t.scalar_type() == torch::kFloat32, name, " must be bf16 or fp32");
}
void chk_f32(const torch::Tensor& t, const char* name) {
  chk(t, name);
  TORCH_CHECK(t.scalar_type() == torch::kFloat32, name, " must be fp32");
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

void scalar_rms_norm(torch::Tensor out, torch::Tensor x, torch::Tensor g, double eps) {
  chk_act(out, "out"); chk_act(x, "x"); chk_f32(g, "g");
  TORCH_CHECK(x.dim() == 2 && out.sizes() == x.sizes() && g.numel() == 1, "scalar_rms_norm: shapes");
  launch_scalar_rms_norm(out.data_ptr(), x.data_ptr(), g.data_ptr<float>(), x.size(0), x.size(1), (float)eps, is_bf(x),
                         is_bf(out), cur());
}

void scalar_norm_add(torch::Tensor res, torch::Tensor y, torch::Tensor g, double eps) {
  chk_f32(res, "res"); chk_act(y, "y"); chk_f32(g, "g");
  TORCH_CHECK(y.dim() == 2 && res.sizes() == y.sizes() && g.numel() == 1, "scalar_norm_add: shapes");
  launch_scalar_norm_add(res.data_ptr<float>(), y.data_ptr(), g.data_ptr<float>(), y.size(0), y.size(1), (float)eps,
                         is_bf(y), cur());
}

// conv [n_slots, 2, keep, W] fp32; slots index its first axis
void chk_conv(const torch::Tensor& conv, const torch::Tensor& w, int64_t W, int64_t sub) {
  chk_f32(conv, "conv"); chk_f32(w, "w");
  TORCH_CHECK(w.dim() == 2 && w.size(0) == W && w.size(1) >= 1 && w.size(1) <= 16, "conv taps must be 1..16, w [W, taps]");
  TORCH_CHECK(conv.dim() == 4 && conv.size(1) == 2 && conv.size(3) == W && conv.size(2) >= std::max<int64_t>(w.size(1) - 1, 1),
              "conv state must be [slots, 2, >= taps - 1, W]");
  TORCH_CHECK(sub == 0 || sub == 1, "sub must be 0 or 1");
}

void canon_norm(torch::Tensor out, torch::Tensor x, torch::Tensor g, double eps, torch::Tensor w, torch::Tensor conv,
                int64_t sub, torch::Tensor row_seq, torch::Tensor positions, torch::Tensor start_pos,
                torch::Tensor slots, bool shift_state) {
  chk_act(out, "out"); chk_f32(x, "x"); chk_f32(g, "g");
  TORCH_CHECK(x.dim() == 2 && out.sizes() == x.sizes() && g.numel() == 1, "canon_norm: shapes");
  const int64_t T = x.size(0), W = x.size(1);
  chk_conv(conv, w, W, sub);
  chk_i32(row_seq, "row_seq", T); chk_i64(positions, "positions", T);
  chk_i32(start_pos, "start_pos"); chk_i32(slots, "slots", start_pos.numel());
  // shifting the state in the same launch is only sound with ONE row per sequence
  TORCH_CHECK(!shift_state || start_pos.numel() == T, "canon_norm: shift_state needs one row per sequence");
  launch_canon_norm(out.data_ptr(), x.data_ptr<float>(), g.data_ptr<float>(), (float)eps, w.data_ptr<float>(),
                    conv.data_ptr<float>(), (int)sub, row_seq.data_ptr<int>(), positions.data_ptr<int64_t>(),
                    start_pos.data_ptr<int>(), slots.data_ptr<int>(), T, W, w.size(1), conv.size(2), is_bf(out), shift_state, cur());
}

void canon_state_update(torch::Tensor x, torch::Tensor g, double eps, torch::Tensor w, torch::Tensor conv, int64_t sub,
                        torch::Tensor cu_q, torch::Tensor start_pos, torch::Tensor slots) {
  chk_f32(x, "x"); chk_f32(g, "g");
  TORCH_CHECK(x.dim() == 2 && g.numel() == 1, "canon_state_update: shapes");
  chk_conv(conv, w, x.size(1), sub);
  const int64_t S = start_pos.numel();
  chk_i32(start_pos, "start_pos"); chk_i32(slots, "slots", S); chk_i32(cu_q, "cu_q", S + 1);
  launch_canon_state(x.data_ptr<float>(), g.data_ptr<float>(), (float)eps, conv.data_ptr<float>(), (int)sub,
                     cu_q.data_ptr<int>(), start_pos.data_ptr<int>(), slots.data_ptr<int>(), S, x.size(1), w.size(1),
                     conv.size(2), cur());
}

void latent_prep(torch::Tensor cq, torch::Tensor proj, int64_t q_rank, int64_t kv_rank, int64_t rot_dim,
                 torch::Tensor wq, torch::Tensor wkv, double eps, torch::Tensor positions, double rot_base,
                 int64_t rot_dims, torch::Tensor cache, torch::Tensor slot_mapping) {
  chk_act(cq, "cq"); chk_act(proj, "proj"); chk_act(cache, "cache"); chk_f32(wq, "wq"); chk_f32(wkv, "wkv");
  TORCH_CHECK(proj.scalar_type() == cq.scalar_type() && proj.scalar_type() == cache.scalar_type(),
              "latent_prep: proj, cq and the cache share one dtype");
  const int64_t T = proj.size(0);
  TORCH_CHECK(proj.dim() == 2 && proj.size(1) >= q_rank + kv_rank + rot_dim, "latent_prep: proj too narrow");
  TORCH_CHECK(cq.dim() == 2 && cq.size(0) == T && cq.size(1) == q_rank, "latent_prep: cq [T, q_rank]");
  TORCH_CHECK(wq.numel() == q_rank && wkv.numel() == kv_rank, "latent_prep: norm weights");
  TORCH_CHECK(cache.dim() == 3 && cache.size(2) == kv_rank + rot_dim, "latent_prep: cache [blocks, BS, kv_rank + rot_dim]");
  TORCH_CHECK(rot_dims >= 0 && rot_dims <= rot_dim && rot_dims % 2 == 0, "latent_prep: rot_dims");
  chk_i64(positions, "positions", T); chk_i64(slot_mapping, "slot_mapping", T);
  launch_latent_prep(cq.data_ptr(), proj.data_ptr(), proj.size(1), T, q_rank, kv_rank, rot_dim, wq.data_ptr<float>(),
                     wkv.data_ptr<float>(), (float)eps, positions.data_ptr<int64_t>(), (float)rot_base, rot_dims,
                     cache.data_ptr(), slot_mapping.data_ptr<int64_t>(), is_bf(proj), cur());
}

void latent_attention(torch::Tensor out, torch::Tensor q_lat, torch::Tensor q, int64_t rot_off, torch::Tensor cache,
                      torch::Tensor block_tables, torch::Tensor cu_q, torch::Tensor start_pos, torch::Tensor tiles,
                      torch::Tensor sink, double scale, double rot_base, int64_t rot_dims, int64_t rows,
                      int64_t num_splits, c10::optional<torch::Tensor> part_o, c10::optional<torch::Tensor> part_ml) {
  chk_act(out, "out"); chk_act(q_lat, "q_lat"); chk_act(q, "q"); chk_act(cache, "cache"); chk_f32(sink, "sink");
  TORCH_CHECK(q_lat.scalar_type() == q.scalar_type() && q.scalar_type() == cache.scalar_type() &&
              out.scalar_type() == q.scalar_type(), "latent_attention: one dtype for q, cache and out");
  TORCH_CHECK(q_lat.dim() == 3 && q.dim() == 3 && cache.dim() == 3, "latent_attention: ranks");
  const int64_t H = q_lat.size(0), T = q_lat.size(1), C = q_lat.size(2);
  const int64_t Dq = q.size(2), R = Dq - rot_off, BS = cache.size(1);
  TORCH_CHECK(q.size(0) == T && q.size(1) == H && rot_off >= 0 && R >= 0, "latent_attention: q [T, H, rot_off + R]");
  TORCH_CHECK(cache.size(2) == C + R, "latent_attention: cache rows must hold C + R = ", C + R, " numbers");
  TORCH_CHECK(out.sizes() == q_lat.sizes() && sink.numel() == H, "latent_attention: out / sink");
  TORCH_CHECK(rot_dims >= 0 && rot_dims <= R && rot_dims % 2 == 0, "latent_attention: rot_dims");
  chk_i32(block_tables, "block_tables"); chk_i32(cu_q, "cu_q"); chk_i32(start_pos, "start_pos", cu_q.numel() - 1);
  chk_i32(tiles, "tiles");
  TORCH_CHECK(block_tables.dim() == 2 && block_tables.size(0) == start_pos.numel(), "latent_attention: block_tables [S, n]");
  TORCH_CHECK(tiles.dim() == 2 && tiles.size(1) == 2, "latent_attention: tiles [n, 2]");
  TORCH_CHECK(num_splits >= 1 && num_splits <= 64, "latent_attention: num_splits must be 1..64");
  float *po = nullptr, *pml = nullptr;
  if (num_splits > 1) {
    TORCH_CHECK(rows == 1, "latent_attention: split keys need one row per tile");
    TORCH_CHECK(part_o.has_value() && part_ml.has_value(), "latent_attention: split keys need the partial buffers");
    chk_f32(*part_o, "part_o"); chk_f32(*part_ml, "part_ml");
    TORCH_CHECK(part_o->numel() >= T * H * num_splits * C && part_ml->numel() >= T * H * num_splits * 2,
                "latent_attention: partial buffers too small");
    po = part_o->data_ptr<float>();
    pml = part_ml->data_ptr<float>();
  }
  int rc = launch_latent_attention(out.data_ptr(), q_lat.data_ptr(), q.data_ptr(), cache.data_ptr(),
                                   block_tables.data_ptr<int>(), cu_q.data_ptr<int>(), start_pos.data_ptr<int>(),
                                   tiles.data_ptr<int>(), tiles.size(0), sink.data_ptr<float>(), po, pml, T, H, C, R, Dq,
                                   rot_off, BS, block_tables.size(1), rows, num_splits, (float)scale, (float)rot_base,
                                   rot_dims, is_bf(q), cur());
  TORCH_CHECK(rc == 0, "latent_attention: unsupported shape (code ", rc, ": 1 rows per tile, 2 latent wider than 512, "
              "3 cached row too wide for the LDS tile)");
}

void gate_mul(torch::Tensor out, torch::Tensor o, torch::Tensor proj, int64_t g_off) {
  chk_act(out, "out"); chk_act(o, "o"); chk_act(proj, "proj");
  TORCH_CHECK(o.dim() == 3 && proj.dim() == 2 && out.dim() == 2, "gate_mul: ranks");
  const int64_t H = o.size(0), T = o.size(1), Dv = o.size(2);
  TORCH_CHECK(out.size(0) == T && out.size(1) == H * Dv && proj.size(0) == T && g_off >= 0 &&
              proj.size(1) >= g_off + H * Dv, "gate_mul: shapes");
  TORCH_CHECK(o.scalar_type() == out.scalar_type() && proj.scalar_type() == out.scalar_type(), "gate_mul: one dtype");
  launch_gate_mul(out.data_ptr(), o.data_ptr(), proj.data_ptr(), proj.size(1), g_off, T, H, Dv, is_bf(out), cur());
}

void poly_norm(torch::Tensor out, torch::Tensor z, torch::Tensor coef, double eps) {
  chk_act(out, "out"); chk_act(z, "z"); chk_f32(coef, "coef");
  TORCH_CHECK(z.dim() == 2 && out.sizes() == z.sizes() && coef.numel() == 4 && out.scalar_type() == z.scalar_type(),
              "poly_norm: shapes");
  launch_poly_norm(out.data_ptr(), z.data_ptr(), coef.data_ptr<float>(), z.size(0), z.size(1), (float)eps, is_bf(z), cur());
}

void logit_softcap(torch::Tensor out, torch::Tensor x, double scale, double cap) {
  chk_f32(out, "out"); chk_act(x, "x");
  TORCH_CHECK(out.numel() == x.numel(), "logit_softcap: shapes");
  launch_softcap(out.data_ptr<float>(), x.data_ptr(), x.numel(), (float)scale, (float)cap, is_bf(x), cur());
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.def("scalar_rms_norm", &scalar_rms_norm);
  m.def("scalar_norm_add", &scalar_norm_add);
  m.def("canon_norm", &canon_norm);
  m.def("canon_state_update", &canon_state_update);
  m.def("latent_prep", &latent_prep);
  m.def("latent_rows_per_tile", [](int64_t H, int64_t C, int64_t R, bool bf) {
    return latent_rows_per_tile((int)H, (int)C, (int)R, bf);
  });
  m.def("latent_attention", &latent_attention);
  m.def("gate_mul", &gate_mul);
  m.def("poly_norm", &poly_norm);
  m.def("logit_softcap", &logit_softcap);
}
