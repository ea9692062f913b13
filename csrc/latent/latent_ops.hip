// L1, L2, L4, L5, L6: the row-wise kernels of the latent-attention model family. All math fp32;
// tensors are bf16 (uint16_t storage) or fp32 as templated. One workgroup per row, about four
// elements per lane (64 .. 1024 lanes); rows are read twice (the second read hits L1 / L2), never staged in LDS, so any row
// width runs.
//
//   scalar_rms_norm   y = x / rms(x) * g                 (g: ONE learned number)
//   scalar_norm_add   res += y / rms(y) * g              (fp32 residual stream, in place)
//   canon_norm        h = x / rms(x) * g ; out = h + sum_j w[:, j] * h_(t - taps + 1 + j)
//                     rows ahead of a sequence's first row of this batch come from its state slot
//   canon_state       shift a sequence's state by its rows of this batch
//   latent_prep       query-latent norm; KV-latent norm + rotary shared key part -> paged cache row
//   gate_mul          [H, T, Dv] head-major -> [T, H * Dv], times sigmoid(gate)
//   poly_norm         a N(z) + b N(z^2) + c N(z^3) + e,  N(u) = u / rms(u)
//   logit_softcap     cap * tanh(scale * x / cap)
#include "../common.h"

namespace {

using rt::DT;
constexpr int kThreads = 256;
constexpr int kMaxTaps = 16;

template <typename IT, typename OT>
__global__ void __launch_bounds__(1024) scalar_rms_norm_kernel(OT* __restrict__ out, const IT* __restrict__ x,
                                                                   const float* __restrict__ g, int W, float eps) {
  __shared__ float scratch[16];
  const IT* xr = x + (size_t)blockIdx.x * W;
  float ss = 0.f;
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    const float v = DT<IT>::load(xr + c);
    ss += v * v;
  }
  const float k = rsqrtf(rt::block_sum(ss, scratch) / W + eps) * g[0];
  OT* o = out + (size_t)blockIdx.x * W;
  for (int c = threadIdx.x; c < W; c += blockDim.x) DT<OT>::store(o + c, DT<IT>::load(xr + c) * k);
}

template <typename IT>
__global__ void __launch_bounds__(1024) scalar_norm_add_kernel(float* __restrict__ res, const IT* __restrict__ y,
                                                                   const float* __restrict__ g, int W, float eps) {
  __shared__ float scratch[16];
  const IT* yr = y + (size_t)blockIdx.x * W;
  float ss = 0.f;
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    const float v = DT<IT>::load(yr + c);
    ss += v * v;
  }
  const float k = rsqrtf(rt::block_sum(ss, scratch) / W + eps) * g[0];
  float* r = res + (size_t)blockIdx.x * W;
  for (int c = threadIdx.x; c < W; c += blockDim.x) r[c] += DT<IT>::load(yr + c) * k;
}

// state layout: conv[slot][sub][i][W], i < keep (= max(taps - 1, 1) allocated rows), oldest first:
// row i of a sequence whose batch starts at position p0 holds the normed input of position
// p0 - (taps - 1) + i.
template <typename OT>
__global__ void __launch_bounds__(1024) canon_norm_kernel(
    OT* __restrict__ out, const float* __restrict__ x, const float* __restrict__ g, float eps,
    const float* __restrict__ w, float* __restrict__ conv, int sub, const int* __restrict__ row_seq,
    const int64_t* __restrict__ positions, const int* __restrict__ start_pos, const int* __restrict__ slots, int W,
    int taps, int keep, int shift_state) {
  __shared__ float scratch[16];
  const int t = blockIdx.x;
  const int s = row_seq[t];
  const int64_t pos = positions[t];
  const int local = (int)(pos - start_pos[s]);
  float* st = conv + ((size_t)slots[s] * 2 + sub) * keep * W;
  // tap k reads the input k rows back: from this batch (local >= k), from the state, or zero
  float inv[kMaxTaps];
  const float* src[kMaxTaps];
  for (int k = 0; k < taps; ++k) {
    inv[k] = 0.f;
    src[k] = nullptr;
    if (local >= k) {
      src[k] = x + (size_t)(t - k) * W;
    } else if (pos >= k) {
      src[k] = st + (size_t)(taps - 1 - k + local) * W;
      inv[k] = 1.f;  // state rows are stored normed
    }
  }
  for (int k = 0; k < taps; ++k) {
    if (local >= k) {
      float ss = 0.f;
      for (int c = threadIdx.x; c < W; c += blockDim.x) {
        const float v = src[k][c];
        ss += v * v;
      }
      inv[k] = rsqrtf(rt::block_sum(ss, scratch) / W + eps) * g[0];
    }
  }
  OT* o = out + (size_t)t * W;
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    const float h0 = src[0][c] * inv[0];
    float acc = h0;
    for (int k = 0; k < taps; ++k)
      if (src[k] != nullptr) acc += w[(size_t)c * taps + (taps - 1 - k)] * (src[k][c] * inv[k]);
    DT<OT>::store(o + c, acc);
    if (shift_state) {
      // one row per sequence (a decode step): this workgroup is the only reader of the sequence's
      // state, and a lane has read its column's old rows above, so it shifts the column here
      for (int i = 0; i + 2 < taps; ++i) st[(size_t)i * W + c] = (pos - (taps - 2 - i) >= 0) ? st[(size_t)(i + 1) * W + c] : 0.f;
      if (taps > 1) st[(size_t)(taps - 2) * W + c] = h0;
    }
  }
}

__global__ void __launch_bounds__(1024) canon_state_kernel(const float* __restrict__ x, const float* __restrict__ g,
                                                               float eps, float* __restrict__ conv, int sub,
                                                               const int* __restrict__ cu_q,
                                                               const int* __restrict__ start_pos,
                                                               const int* __restrict__ slots, int W, int taps, int keep) {
  __shared__ float scratch[16];
  const int s = blockIdx.x;
  const int r0 = cu_q[s], n = cu_q[s + 1] - r0;
  if (n <= 0) return;
  const int kn = taps - 1;
  float* st = conv + ((size_t)slots[s] * 2 + sub) * keep * W;
  float inv[kMaxTaps];
  for (int i = 0; i < kn; ++i) {
    const int idx = n - kn + i;  // row of this batch, or (< 0) a row of the old state
    inv[i] = 0.f;
    if (idx >= 0) {
      const float* xr = x + (size_t)(r0 + idx) * W;
      float ss = 0.f;
      for (int c = threadIdx.x; c < W; c += blockDim.x) ss += xr[c] * xr[c];
      inv[i] = rsqrtf(rt::block_sum(ss, scratch) / W + eps) * g[0];
    }
  }
  const int p0 = start_pos[s];
  // a lane owns its columns: it reads every old row of a column before it writes the new ones
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    float nv[kMaxTaps];
    for (int i = 0; i < kn; ++i) {
      const int idx = n - kn + i;
      if (idx >= 0) nv[i] = x[(size_t)(r0 + idx) * W + c] * inv[i];
      else if (p0 + idx >= 0) nv[i] = st[(size_t)(kn + idx) * W + c];
      else nv[i] = 0.f;
    }
    for (int i = 0; i < kn; ++i) st[(size_t)i * W + c] = nv[i];
  }
}

// rotary frequency of pair i: base^(-2i / dims), as exp2 of a product (the PyTorch statement of
// the op computes the same expression)
RT_DEVICE float rot_freq(int i, float neg2_log2base_over_dims) { return exp2f((float)i * neg2_log2base_over_dims); }

template <typename PT, typename CT, typename OT>
__global__ void __launch_bounds__(1024) latent_prep_kernel(
    OT* __restrict__ cq, const PT* __restrict__ proj, int proj_stride, int q_rank, int kv_rank, int rot_dim,
    const float* __restrict__ wq, const float* __restrict__ wkv, float eps, const int64_t* __restrict__ positions,
    float rot_k, int rot_dims, CT* __restrict__ cache, const int64_t* __restrict__ slot_mapping) {
  __shared__ float scratch[16];
  const int t = blockIdx.x;
  const PT* p = proj + (size_t)t * proj_stride;
  float sq = 0.f, sk = 0.f;
  for (int c = threadIdx.x; c < q_rank; c += blockDim.x) {
    const float v = DT<PT>::load(p + c);
    sq += v * v;
  }
  for (int c = threadIdx.x; c < kv_rank; c += blockDim.x) {
    const float v = DT<PT>::load(p + q_rank + c);
    sk += v * v;
  }
  const float iq = rsqrtf(rt::block_sum(sq, scratch) / q_rank + eps);
  const float ik = rsqrtf(rt::block_sum(sk, scratch) / kv_rank + eps);
  OT* o = cq + (size_t)t * q_rank;
  for (int c = threadIdx.x; c < q_rank; c += blockDim.x) DT<OT>::store(o + c, DT<PT>::load(p + c) * iq * wq[c]);
  CT* row = cache + (size_t)slot_mapping[t] * (kv_rank + rot_dim);
  for (int c = threadIdx.x; c < kv_rank; c += blockDim.x)
    DT<CT>::store(row + c, DT<PT>::load(p + q_rank + c) * ik * wkv[c]);
  const PT* pr = p + q_rank + kv_rank;
  const float posf = (float)positions[t];
  for (int i = threadIdx.x; i < rot_dim / 2 + (rot_dim & 1); i += blockDim.x) {
    const float u = DT<PT>::load(pr + 2 * i);
    if (2 * i + 1 >= rot_dim) {  // odd tail entry: never rotated
      DT<CT>::store(row + kv_rank + 2 * i, u);
      continue;
    }
    const float v = DT<PT>::load(pr + 2 * i + 1);
    float cs = 1.f, sn = 0.f;
    if (2 * i < rot_dims) sincosf(posf * rot_freq(i, rot_k), &sn, &cs);
    DT<CT>::store(row + kv_rank + 2 * i, u * cs - v * sn);
    DT<CT>::store(row + kv_rank + 2 * i + 1, v * cs + u * sn);
  }
}

template <typename IT, typename PT, typename OT>
__global__ void __launch_bounds__(1024) gate_mul_kernel(OT* __restrict__ out, const IT* __restrict__ o,
                                                            const PT* __restrict__ proj, int proj_stride, int g_off,
                                                            int T, int H, int Dv) {
  const int t = blockIdx.x;
  const int n = H * Dv;
  for (int c = threadIdx.x; c < n; c += blockDim.x) {
    const int h = c / Dv, d = c - h * Dv;
    const float v = DT<IT>::load(o + ((size_t)h * T + t) * Dv + d);
    const float gt = DT<PT>::load(proj + (size_t)t * proj_stride + g_off + c);
    DT<OT>::store(out + (size_t)t * n + c, v / (1.f + expf(-gt)));
  }
}

template <typename IT, typename OT>
__global__ void __launch_bounds__(1024) poly_norm_kernel(OT* __restrict__ out, const IT* __restrict__ z,
                                                             const float* __restrict__ coef, int F, float eps) {
  __shared__ float scratch[16];
  const IT* zr = z + (size_t)blockIdx.x * F;
  float s1 = 0.f, s2 = 0.f, s3 = 0.f;
  for (int c = threadIdx.x; c < F; c += blockDim.x) {
    const float v = DT<IT>::load(zr + c);
    const float v2 = v * v;
    s1 += v2;
    s2 += v2 * v2;
    s3 += v2 * v2 * v2;
  }
  const float k1 = coef[0] * rsqrtf(rt::block_sum(s1, scratch) / F + eps);
  const float k2 = coef[1] * rsqrtf(rt::block_sum(s2, scratch) / F + eps);
  const float k3 = coef[2] * rsqrtf(rt::block_sum(s3, scratch) / F + eps);
  const float e = coef[3];
  OT* o = out + (size_t)blockIdx.x * F;
  for (int c = threadIdx.x; c < F; c += blockDim.x) {
    const float v = DT<IT>::load(zr + c);
    DT<OT>::store(o + c, k1 * v + k2 * (v * v) + k3 * (v * v * v) + e);
  }
}

template <typename IT>
__global__ void __launch_bounds__(kThreads) softcap_kernel(float* __restrict__ out, const IT* __restrict__ x, int64_t n,
                                                           float scale, float cap) {
  const int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  if (i >= n) return;
  const float v = DT<IT>::load(x + i) * scale;
  out[i] = cap > 0.f ? cap * tanhf(v / cap) : v;
}

}  // namespace

// ---- launchers: `bf` flags say which operands are bf16 (else fp32) -----------------------------
// lanes per row: about four elements each, whole waves, at most 1024 (wide rows of a decode step
// are latency-bound: few workgroups, so each one spreads its row over many lanes)
static int row_threads(int W) {
  int t = ((W + 3) / 4 + 63) / 64 * 64;
  return t < 64 ? 64 : t > 1024 ? 1024 : t;
}
#define RT_LAUNCH_W(kern, grid, W, ...) hipLaunchKernelGGL(kern, dim3(grid), dim3(row_threads(W)), 0, stream, __VA_ARGS__)
#define RT_LAUNCH(kern, grid, ...) hipLaunchKernelGGL(kern, dim3(grid), dim3(kThreads), 0, stream, __VA_ARGS__)

void launch_scalar_rms_norm(void* out, const void* x, const float* g, int rows, int W, float eps, bool in_bf,
                            bool out_bf, hipStream_t stream) {
  if (rows <= 0) return;
  if (in_bf && out_bf) RT_LAUNCH_W((scalar_rms_norm_kernel<uint16_t, uint16_t>), rows, W, (uint16_t*)out, (const uint16_t*)x, g, W, eps);
  else if (in_bf) RT_LAUNCH_W((scalar_rms_norm_kernel<uint16_t, float>), rows, W, (float*)out, (const uint16_t*)x, g, W, eps);
  else if (out_bf) RT_LAUNCH_W((scalar_rms_norm_kernel<float, uint16_t>), rows, W, (uint16_t*)out, (const float*)x, g, W, eps);
  else RT_LAUNCH_W((scalar_rms_norm_kernel<float, float>), rows, W, (float*)out, (const float*)x, g, W, eps);
}

void launch_scalar_norm_add(float* res, const void* y, const float* g, int rows, int W, float eps, bool y_bf,
                            hipStream_t stream) {
  if (rows <= 0) return;
  if (y_bf) RT_LAUNCH_W((scalar_norm_add_kernel<uint16_t>), rows, W, res, (const uint16_t*)y, g, W, eps);
  else RT_LAUNCH_W((scalar_norm_add_kernel<float>), rows, W, res, (const float*)y, g, W, eps);
}

void launch_canon_norm(void* out, const float* x, const float* g, float eps, const float* w, float* conv, int sub,
                       const int* row_seq, const int64_t* positions, const int* start_pos, const int* slots, int T,
                       int W, int taps, int keep, bool out_bf, bool shift_state, hipStream_t stream) {
  if (T <= 0) return;
  if (out_bf) RT_LAUNCH_W((canon_norm_kernel<uint16_t>), T, W, (uint16_t*)out, x, g, eps, w, conv, sub, row_seq, positions, start_pos, slots, W, taps, keep, shift_state ? 1 : 0);
  else RT_LAUNCH_W((canon_norm_kernel<float>), T, W, (float*)out, x, g, eps, w, conv, sub, row_seq, positions, start_pos, slots, W, taps, keep, shift_state ? 1 : 0);
}

void launch_canon_state(const float* x, const float* g, float eps, float* conv, int sub, const int* cu_q,
                        const int* start_pos, const int* slots, int S, int W, int taps, int keep, hipStream_t stream) {
  if (S <= 0 || taps <= 1) return;
  RT_LAUNCH_W(canon_state_kernel, S, W, x, g, eps, conv, sub, cu_q, start_pos, slots, W, taps, keep);
}

void launch_latent_prep(void* cq, const void* proj, int proj_stride, int T, int q_rank, int kv_rank, int rot_dim,
                        const float* wq, const float* wkv, float eps, const int64_t* positions, float rot_base,
                        int rot_dims, void* cache, const int64_t* slot_mapping, bool bf, hipStream_t stream) {
  if (T <= 0) return;
  const float rot_k = rot_dims > 0 ? -2.0f * log2f(rot_base) / (float)rot_dims : 0.f;
  if (bf) RT_LAUNCH_W((latent_prep_kernel<uint16_t, uint16_t, uint16_t>), T, (q_rank > kv_rank ? q_rank : kv_rank), (uint16_t*)cq, (const uint16_t*)proj, proj_stride, q_rank, kv_rank, rot_dim, wq, wkv, eps, positions, rot_k, rot_dims, (uint16_t*)cache, slot_mapping);
  else RT_LAUNCH_W((latent_prep_kernel<float, float, float>), T, (q_rank > kv_rank ? q_rank : kv_rank), (float*)cq, (const float*)proj, proj_stride, q_rank, kv_rank, rot_dim, wq, wkv, eps, positions, rot_k, rot_dims, (float*)cache, slot_mapping);
}

void launch_gate_mul(void* out, const void* o, const void* proj, int proj_stride, int g_off, int T, int H, int Dv,
                     bool bf, hipStream_t stream) {
  if (T <= 0) return;
  if (bf) RT_LAUNCH_W((gate_mul_kernel<uint16_t, uint16_t, uint16_t>), T, H * Dv, (uint16_t*)out, (const uint16_t*)o, (const uint16_t*)proj, proj_stride, g_off, T, H, Dv);
  else RT_LAUNCH_W((gate_mul_kernel<float, float, float>), T, H * Dv, (float*)out, (const float*)o, (const float*)proj, proj_stride, g_off, T, H, Dv);
}

void launch_poly_norm(void* out, const void* z, const float* coef, int rows, int F, float eps, bool bf,
                      hipStream_t stream) {
  if (rows <= 0) return;
  if (bf) RT_LAUNCH_W((poly_norm_kernel<uint16_t, uint16_t>), rows, F, (uint16_t*)out, (const uint16_t*)z, coef, F, eps);
  else RT_LAUNCH_W((poly_norm_kernel<float, float>), rows, F, (float*)out, (const float*)z, coef, F, eps);
}

void launch_softcap(float* out, const void* x, int64_t n, float scale, float cap, bool bf, hipStream_t stream) {
  if (n <= 0) return;
  const int grid = (int)((n + kThreads - 1) / kThreads);
  if (bf) RT_LAUNCH((softcap_kernel<uint16_t>), grid, out, (const uint16_t*)x, n, scale, cap);
  else RT_LAUNCH((softcap_kernel<float>), grid, out, (const float*)x, n, scale, cap);
}
