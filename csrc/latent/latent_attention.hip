// L3: causal attention over the paged latent cache with a softmax sink, for any head count and
// any latent / rotary width (fp32 FMA; the cache and queries are bf16 or fp32 as templated).
//
// The query of every head has been folded into latent space (q_lat = q_unrotated . W_uk), so the
// key of token t is its cached row [latent C | rotated key part R] and its value is the row's
// first C entries: ALL heads read the SAME rows. One workgroup (4 waves) takes a tile of query
// rows of one sequence with all their heads ("pairs" = rows x heads, PW per wave) and walks the
// sequence's keys 64 at a time:
//
//   stage   the 64 cached rows (paged: block table lookup per key) into LDS, once for all pairs
//   scores  lane = key: s[p] = sum_d q[p][d] * K[key][d]   (q in LDS, read as a broadcast)
//   softmax online per pair (running max m, sum l), masked by each row's own position
//   values  lane = latent column: o[p][c] += sum_key p[key] * K[key][c]   (P via LDS)
//
// The sink enters once, at the end: the denominator gains exp(sink_h - m). With `num_splits` > 1
// (one query row per sequence: the decode step) a workgroup takes one contiguous range of each
// tile's keys and writes (o, m, l) partials that `latent_combine_kernel` merges; the ranges
// follow from the run-time position, so one captured launch serves every length.
//
// The rotary part of q is rotated here, on load, by the row's position (fp32 angles).
#include <cstdlib>

#include "../common.h"

namespace {

using rt::DT;
constexpr int kWaves = 4;
constexpr int kThreads = kWaves * 64;
constexpr int KT = 64;  // keys per tile: one per lane

struct AttnArgs {
  void* out;            // [H, T, C]
  const void* q_lat;    // [H, T, C]
  const void* q;        // [T, H, Dq]; entries rot_off.. of a head are its rotary part
  const void* cache;    // [num_blocks, BS, Dk], Dk = C + R
  const int* block_tables;
  const int* cu_q;
  const int* start_pos;
  const int* tiles;     // [n_tiles, 2] (sequence, first row)
  const float* sink;    // [H]
  float* part_o;        // [T, H, splits, C]
  float* part_ml;       // [T, H, splits, 2]
  int T, H, C, R, Dq, rot_off, BS, max_blocks, rows, num_splits, kstride, rot_dims;
  int hwin;             // heads one workgroup takes (grid.z walks the windows)
  int kt;               // keys per staged tile of the plain kernel (64, or fewer when LDS is short)
  float scale, rot_k;
};

// CPL: latent columns per lane (C <= 64 * CPL); PW: (row, head) pairs per wave
template <typename CT, typename QT, int CPL, int PW>
__global__ void __launch_bounds__(kThreads) latent_attn_kernel(AttnArgs a) {
  extern __shared__ __align__(16) unsigned char smem[];
  const int Dk = a.C + a.R;
  CT* Ks = reinterpret_cast<CT*>(smem);                                   // [kt][kstride]
  float* Qs = reinterpret_cast<float*>(smem + (size_t)a.kt * a.kstride * sizeof(CT));  // [pairs][Dk]
  float* Ps = Qs + (size_t)kWaves * PW * Dk;                              // [pairs][KT]
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int seq = a.tiles[blockIdx.x * 2], row0 = a.tiles[blockIdx.x * 2 + 1];
  const int nrows = min(a.rows, a.cu_q[seq + 1] - row0);
  const int pos0 = a.start_pos[seq] + (row0 - a.cu_q[seq]);   // position of the tile's first row
  const int h0 = blockIdx.z * a.hwin;
  const int HW = min(a.hwin, a.H - h0);     // heads of this workgroup's window
  const int npairs = nrows * HW;
  // this wave's pairs: p = wave * PW + i -> (row p / HW, head h0 + p % HW)
  // ---- queries -> LDS (scaled; rotary part rotated by the row's position) ----
  for (int p = wave; p < kWaves * PW; p += kWaves) {
    float* qd = Qs + (size_t)p * Dk;
    if (p >= npairs) {
      for (int d = lane; d < Dk; d += 64) qd[d] = 0.f;
      continue;
    }
    const int r = p / HW, h = h0 + p - r * HW;
    const QT* ql = reinterpret_cast<const QT*>(a.q_lat) + ((size_t)h * a.T + row0 + r) * a.C;
    for (int d = lane; d < a.C; d += 64) qd[d] = DT<QT>::load(ql + d) * a.scale;
    const QT* qr = reinterpret_cast<const QT*>(a.q) + ((size_t)(row0 + r) * a.H + h) * a.Dq + a.rot_off;
    const float posf = (float)(pos0 + r);
    for (int i = lane; i < (a.R + 1) / 2; i += 64) {
      const float u = DT<QT>::load(qr + 2 * i);
      if (2 * i + 1 >= a.R) {
        qd[a.C + 2 * i] = u * a.scale;
        continue;
      }
      const float v = DT<QT>::load(qr + 2 * i + 1);
      float cs = 1.f, sn = 0.f;
      if (2 * i < a.rot_dims) sincosf(posf * exp2f((float)i * a.rot_k), &sn, &cs);
      qd[a.C + 2 * i] = (u * cs - v * sn) * a.scale;
      qd[a.C + 2 * i + 1] = (v * cs + u * sn) * a.scale;
    }
  }
  float m[PW], l[PW], o[PW][CPL];
  int qpos[PW];
#pragma unroll
  for (int i = 0; i < PW; ++i) {
    m[i] = -INFINITY;
    l[i] = 0.f;
    const int p = wave * PW + i;
    qpos[i] = p < npairs ? pos0 + p / HW : -1;   // -1: no key is visible, the pair stays empty
#pragma unroll
    for (int j = 0; j < CPL; ++j) o[i][j] = 0.f;
  }
  // ---- key range of this workgroup ----
  const int nkeys = pos0 + nrows;   // keys 0 .. last row's position
  int kb = 0, ke = nkeys;
  if (a.num_splits > 1) {
    const int ntile = (nkeys + KT - 1) / KT;
    const int per = (ntile + a.num_splits - 1) / a.num_splits;
    kb = min(nkeys, (int)blockIdx.y * per * KT);
    ke = min(nkeys, kb + per * KT);
  }
  const int* bt = a.block_tables + (size_t)seq * a.max_blocks;
  const CT* cache = reinterpret_cast<const CT*>(a.cache);
  const int kt = a.kt;
  for (int k0 = kb; k0 < ke; k0 += kt) {
    __syncthreads();   // the previous tile's readers are done (and Qs is written, first time)
    // stage: wave w copies keys w, w + 4, ...; lanes stride over the row
    for (int kk = wave; kk < kt; kk += kWaves) {
      const int kp = k0 + kk;
      CT* dst = Ks + (size_t)kk * a.kstride;
      if (kp < ke) {
        const CT* src = cache + ((size_t)bt[kp / a.BS] * a.BS + kp % a.BS) * Dk;
        for (int d = lane; d < Dk; d += 64) dst[d] = src[d];
      } else {
        for (int d = lane; d < Dk; d += 64) dst[d] = CT(0);
      }
    }
    __syncthreads();
    // scores: lane = key
    float s[PW];
#pragma unroll
    for (int i = 0; i < PW; ++i) s[i] = 0.f;
    const CT* krow = Ks + (size_t)(lane < kt ? lane : 0) * a.kstride;
    const float* qw = Qs + (size_t)wave * PW * Dk;
    for (int d = 0; d < Dk; ++d) {
      const float kv = DT<CT>::load(krow + d);
#pragma unroll
      for (int i = 0; i < PW; ++i) s[i] += qw[(size_t)i * Dk + d] * kv;
    }
    const int kp = k0 + lane;
    float* pw = Ps + (size_t)wave * PW * KT;
#pragma unroll
    for (int i = 0; i < PW; ++i) {
      const bool vis = lane < kt && kp < ke && kp <= qpos[i];
      const float sv = vis ? s[i] : -INFINITY;
      const float mn = fmaxf(m[i], rt::wave_max(sv));
      float p = 0.f, alpha = 1.f;
      if (mn > -INFINITY) {
        p = vis ? __expf(sv - mn) : 0.f;
        alpha = __expf(m[i] - mn);   // m = -inf -> 0
      }
      l[i] = l[i] * alpha + rt::wave_sum(p);
      m[i] = mn;
#pragma unroll
      for (int j = 0; j < CPL; ++j) o[i][j] *= alpha;
      pw[i * KT + lane] = p;
    }
    // values: lane = latent column(s); P is read back as a broadcast (same wave wrote it)
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    for (int kk = 0; kk < kt; ++kk) {
      float kvv[CPL];
#pragma unroll
      for (int j = 0; j < CPL; ++j) {
        const int c = lane + 64 * j;
        kvv[j] = c < a.C ? DT<CT>::load(Ks + (size_t)kk * a.kstride + c) : 0.f;
      }
#pragma unroll
      for (int i = 0; i < PW; ++i) {
        const float p = pw[i * KT + kk];
#pragma unroll
        for (int j = 0; j < CPL; ++j) o[i][j] += p * kvv[j];
      }
    }
  }
  // ---- finish: the sink joins the denominator (single launch) or partials go to the combine ----
#pragma unroll
  for (int i = 0; i < PW; ++i) {
    const int p = wave * PW + i;
    if (p >= npairs) continue;
    const int r = p / HW, h = h0 + p - r * HW;
    const int t = row0 + r;
    if (a.num_splits > 1) {
      float* po = a.part_o + (((size_t)t * a.H + h) * a.num_splits + blockIdx.y) * a.C;
#pragma unroll
      for (int j = 0; j < CPL; ++j) {
        const int c = lane + 64 * j;
        if (c < a.C) po[c] = o[i][j];
      }
      if (lane == 0) {
        float* ml = a.part_ml + (((size_t)t * a.H + h) * a.num_splits + blockIdx.y) * 2;
        ml[0] = m[i];
        ml[1] = l[i];
      }
    } else {
      const float sk = a.sink[h];
      const float M = fmaxf(m[i], sk);
      const float w = __expf(m[i] - M);
      const float inv = 1.f / (l[i] * w + __expf(sk - M));
      CT* orow = reinterpret_cast<CT*>(a.out) + ((size_t)h * a.T + t) * a.C;
#pragma unroll
      for (int j = 0; j < CPL; ++j) {
        const int c = lane + 64 * j;
        if (c < a.C) DT<CT>::store(orow + c, o[i][j] * w * inv);
      }
    }
  }
}

// one workgroup per (row, head): merge the split partials and the sink. The splits' weights are
// formed once (LDS), then every lane sums its columns over the splits with coalesced loads.
template <typename OT>
__global__ void __launch_bounds__(256) latent_combine_kernel(OT* __restrict__ out, const float* __restrict__ part_o,
                                                             const float* __restrict__ part_ml,
                                                             const float* __restrict__ sink, int T, int H, int C,
                                                             int splits) {
  __shared__ float wgt[64];
  __shared__ float inv_s;
  const int t = blockIdx.x, h = blockIdx.y;
  const float* ml = part_ml + ((size_t)t * H + h) * splits * 2;
  if (threadIdx.x < 64) {
    const int s = threadIdx.x;
    const float sk = sink[h];
    const float ms = s < splits ? ml[2 * s] : -INFINITY;
    const float M = fmaxf(rt::wave_max(ms), sk);
    const float w = s < splits ? __expf(ms - M) : 0.f;          // m = -inf (an empty split) -> 0
    const float den = rt::wave_sum(s < splits ? ml[2 * s + 1] * w : 0.f) + __expf(sk - M);
    wgt[s] = w;
    if (s == 0) inv_s = 1.f / den;
  }
  __syncthreads();
  const float inv = inv_s;
  const float* po = part_o + ((size_t)t * H + h) * splits * C;
  OT* orow = out + ((size_t)h * T + t) * C;
  for (int c = threadIdx.x; c < C; c += blockDim.x) {
    float acc = 0.f;
    for (int s = 0; s < splits; ++s) {
      const float w = wgt[s];
      if (w > 0.f) acc += po[(size_t)s * C + c] * w;
    }
    DT<OT>::store(orow + c, acc * inv);
  }
}

// ---- bf16 on the matrix cores ----------------------------------------------------------------
// Workgroup = 4 waves over 64 (row, head) pairs and a 64-key tile; wave w = (ph, x): ph = w >> 1
// is its half of the pairs (32 MFMA columns), x = w & 1 its half of the tile's KEYS while scores
// are formed and its half of the latent COLUMNS while values are accumulated:
//
//   stage    lane = key: the tile's rows -> LDS row-major (K), and their latent part transposed
//            (V^T [C][64 keys]): the value product contracts over keys, the cache row over dims
//   S^T      [32 keys x 32 pairs] = K . Q^T   Dk/16 x mfma_f32_32x32x16_bf16, Q fragments in
//            registers; K rows are read with bits 2 and 3 of the row index swapped, which leaves
//            lane (pair, h) with keys 16j + 8h + 0..7: the B fragment of P^T as it stands
//   softmax  each lane owns ONE pair: mask by its position, tile maximum over the wave's keys,
//            exchanged with the other key half through LDS, P -> LDS [pair][key] as bf16
//   O^T      [C/2 latent cols x 32 pairs] += V^T . P^T   (C/64 blocks x 4 key chunks)
//
// Needs C a multiple of 64 (<= 512), R a multiple of 16 (<= 64).
typedef float f16v __attribute__((ext_vector_type(16)));
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;
#ifndef RT_STAGE_BATCH
#define RT_STAGE_BATCH 9
#endif
constexpr int kStageBatch = RT_STAGE_BATCH;   // staging loads in flight per lane
constexpr int kVRow = KT * 2 + 16;   // bytes per V^T / P row in LDS (64 keys + pad)

RT_DEVICE int swap23(int x) { return (x & ~12) | ((x & 4) << 1) | ((x & 8) >> 1); }

template <int NB>   // NB = C / 64: 32-column value blocks per wave
__global__ void __launch_bounds__(kThreads) latent_attn_mfma_kernel(AttnArgs a) {
  constexpr int NQM = NB * 4 + 4;
  extern __shared__ __align__(16) unsigned char smem[];
  const int C = a.C, Dk = a.C + a.R, nq = Dk >> 4;
  const int krow_b = Dk * 2 + 16;
  unsigned char* Kt = smem;
  unsigned char* Vt = Kt + (size_t)KT * krow_b;
  unsigned char* Pt = Vt + (size_t)C * kVRow;
  float* mx = reinterpret_cast<float*>(Pt + 64 * kVRow);   // [2][64]
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int c = lane & 31, h = lane >> 5, ph = wave >> 1, x = wave & 1;
  const int seq = a.tiles[blockIdx.x * 2], row0 = a.tiles[blockIdx.x * 2 + 1];
  const int nrows = min(a.rows, a.cu_q[seq + 1] - row0);
  const int pos0 = a.start_pos[seq] + (row0 - a.cu_q[seq]);
  const int h0 = blockIdx.z * a.hwin;
  const int HW = min(a.hwin, a.H - h0);
  const int npairs = nrows * HW;
  // ---- queries -> LDS (bf16, rotary part rotated), then each lane's B fragments -> registers ----
  for (int p = wave; p < 64; p += kWaves) {
    uint16_t* qd = reinterpret_cast<uint16_t*>(Kt + (size_t)p * krow_b);
    if (p >= npairs) {
      for (int d = lane; d < Dk; d += 64) qd[d] = 0;
      continue;
    }
    const int r = p / HW, hd = h0 + p - r * HW;
    const uint16_t* ql = reinterpret_cast<const uint16_t*>(a.q_lat) + ((size_t)hd * a.T + row0 + r) * C;
    for (int d = lane; d < C; d += 64) qd[d] = ql[d];
    const uint16_t* qr = reinterpret_cast<const uint16_t*>(a.q) + ((size_t)(row0 + r) * a.H + hd) * a.Dq + a.rot_off;
    const float posf = (float)(pos0 + r);
    for (int i = lane; i < a.R / 2; i += 64) {
      const float u = rt::bf2f(qr[2 * i]), v = rt::bf2f(qr[2 * i + 1]);
      float cs = 1.f, sn = 0.f;
      if (2 * i < a.rot_dims) sincosf(posf * exp2f((float)i * a.rot_k), &sn, &cs);
      qd[C + 2 * i] = rt::f2bf(u * cs - v * sn);
      qd[C + 2 * i + 1] = rt::f2bf(v * cs + u * sn);
    }
  }
  __syncthreads();
  rt::short8 qf[NQM];
#pragma unroll
  for (int dk = 0; dk < NQM; ++dk)
    if (dk < nq) qf[dk] = *reinterpret_cast<const rt::short8*>(Kt + (size_t)(ph * 32 + c) * krow_b + 32 * dk + 16 * h);
  const int mp = ph * 32 + c;                              // this lane's pair
  const int qpos = mp < npairs ? pos0 + mp / HW : -1;
  f16v o[NB];
#pragma unroll
  for (int db = 0; db < NB; ++db)
#pragma unroll
    for (int i = 0; i < 16; ++i) o[db][i] = 0.f;
  float m = -INFINITY, l = 0.f;   // m in log2 units of the scaled score
  const float sc2 = a.scale * kLog2e;
  const int nkeys = pos0 + nrows;
  int kb = 0, ke = nkeys;
  if (a.num_splits > 1) {
    const int ntile = (nkeys + KT - 1) / KT;
    const int per = (ntile + a.num_splits - 1) / a.num_splits;
    kb = min(nkeys, (int)blockIdx.y * per * KT);
    ke = min(nkeys, kb + per * KT);
  }
  const int* bt = a.block_tables + (size_t)seq * a.max_blocks;
  const uint16_t* cache = reinterpret_cast<const uint16_t*>(a.cache);
  const int nch = Dk >> 3;   // 16-byte chunks per cached row
  for (int k0 = kb; k0 < ke; k0 += KT) {
    __syncthreads();   // the previous tile (and the query fragments' source) is consumed
    {
      const int kp = k0 + lane;
      const bool ok = kp < ke;
      const uint16_t* src = cache + ((size_t)(ok ? bt[kp / a.BS] : 0) * a.BS + (ok ? kp % a.BS : 0)) * Dk;
      // a batch of chunk loads is issued before the first is consumed
      auto put = [&](int ch, const rt::u32x4& v) {
        *reinterpret_cast<rt::u32x4*>(Kt + (size_t)lane * krow_b + ch * 16) = v;
        if (ch * 8 < C) {
          uint16_t* vt = reinterpret_cast<uint16_t*>(Vt + (size_t)(ch * 8) * kVRow) + lane;
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            vt[(size_t)(2 * j) * (kVRow / 2)] = (uint16_t)(v[j] & 0xffffu);
            vt[(size_t)(2 * j + 1) * (kVRow / 2)] = (uint16_t)(v[j] >> 16);
          }
        }
      };
      for (int ch = wave; ch < nch; ch += kStageBatch * kWaves) {
        rt::u32x4 v[kStageBatch];
#pragma unroll
        for (int u = 0; u < kStageBatch; ++u) {
          v[u] = rt::u32x4{0u, 0u, 0u, 0u};
          const int cu_ = ch + u * kWaves;
          if (ok && cu_ < nch) v[u] = *reinterpret_cast<const rt::u32x4*>(src + cu_ * 8);
        }
#pragma unroll
        for (int u = 0; u < kStageBatch; ++u) {
          const int cu_ = ch + u * kWaves;
          if (cu_ < nch) put(cu_, v[u]);
        }
      }
    }
    __syncthreads();
    // ---- S^T = K Q^T for this wave's 32 keys x 32 pairs ----
    f16v sc;
#pragma unroll
    for (int i = 0; i < 16; ++i) sc[i] = 0.f;
    const unsigned char* kr = Kt + (size_t)(32 * x + swap23(c)) * krow_b + 16 * h;
#pragma unroll
    for (int dk = 0; dk < NQM; ++dk)
      if (dk < nq) {
        const rt::short8 ka = *reinterpret_cast<const rt::short8*>(kr + 32 * dk);
        sc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(rt::bf16x8, ka),
                                                     __builtin_bit_cast(rt::bf16x8, qf[dk]), sc, 0, 0, 0);
      }
    // reg i holds key k0 + 32x + 16 (i >> 3) + 8h + (i & 7) of pair mp
    float tmax = -INFINITY;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int key = k0 + 32 * x + 16 * (i >> 3) + 8 * h + (i & 7);
      const float v = (key < ke && key <= qpos) ? sc[i] * sc2 : -INFINITY;
      sc[i] = v;
      tmax = fmaxf(tmax, v);
    }
    tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
    if (h == 0) mx[x * 64 + mp] = tmax;
    __syncthreads();
    const float mn = fmaxf(m, fmaxf(mx[mp], mx[64 + mp]));
    const float msub = (mn == -INFINITY) ? 0.f : mn;
    const float alpha = (mn == -INFINITY) ? 1.f : exp2f(m - mn);
    m = mn;
    float psum = 0.f;
#pragma unroll
    for (int blk = 0; blk < 2; ++blk) {
      rt::u32x4 w;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float p0 = exp2f(sc[8 * blk + 2 * j] - msub), p1 = exp2f(sc[8 * blk + 2 * j + 1] - msub);
        psum += p0 + p1;
        w[j] = rt::pack2(p0, p1);
      }
      *reinterpret_cast<rt::u32x4*>(Pt + (size_t)mp * kVRow + (32 * x + 16 * blk + 8 * h) * 2) = w;
    }
    l = l * alpha + psum;
#pragma unroll
    for (int db = 0; db < NB; ++db)
#pragma unroll
      for (int i = 0; i < 16; ++i) o[db][i] *= alpha;
    __syncthreads();
    // ---- O^T += V^T P^T for this wave's half of the latent columns ----
    const unsigned char* pr = Pt + (size_t)mp * kVRow + 16 * h;
#pragma unroll
    for (int db = 0; db < NB; ++db) {
      const unsigned char* vr = Vt + (size_t)(x * (C / 2) + 32 * db + c) * kVRow + 16 * h;
#pragma unroll
      for (int kc = 0; kc < 4; ++kc) {
        const rt::short8 va = *reinterpret_cast<const rt::short8*>(vr + 32 * kc);
        const rt::short8 pb = *reinterpret_cast<const rt::short8*>(pr + 32 * kc);
        o[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(rt::bf16x8, va),
                                                        __builtin_bit_cast(rt::bf16x8, pb), o[db], 0, 0, 0);
      }
    }
  }
  // ---- the pair's sum over both key halves, then the sink (or the split partials) ----
  l += __shfl_xor(l, 32, 64);
  __syncthreads();
  if (h == 0) mx[x * 64 + mp] = l;
  __syncthreads();
  const float ltot = mx[mp] + mx[64 + mp];
  if (mp >= npairs) return;
  const int r = mp / HW, hd = h0 + mp - r * HW, t = row0 + r;
  const float m_nat = m * kLn2;
  if (a.num_splits > 1) {
    float* po = a.part_o + (((size_t)t * a.H + hd) * a.num_splits + blockIdx.y) * C;
#pragma unroll
    for (int db = 0; db < NB; ++db)
#pragma unroll
      for (int i = 0; i < 16; ++i) po[x * (C / 2) + 32 * db + 8 * (i >> 2) + 4 * h + (i & 3)] = o[db][i];
    if (x == 0 && h == 0) {
      float* ml = a.part_ml + (((size_t)t * a.H + hd) * a.num_splits + blockIdx.y) * 2;
      ml[0] = m_nat;
      ml[1] = ltot;
    }
  } else {
    const float sk = a.sink[hd];
    const float M = fmaxf(m_nat, sk);
    const float w = __expf(m_nat - M);
    const float inv = w / (ltot * w + __expf(sk - M));
    uint16_t* orow = reinterpret_cast<uint16_t*>(a.out) + ((size_t)hd * a.T + t) * C;
#pragma unroll
    for (int db = 0; db < NB; ++db)
#pragma unroll
      for (int i = 0; i < 16; ++i)
        orow[x * (C / 2) + 32 * db + 8 * (i >> 2) + 4 * h + (i & 3)] = rt::f2bf(o[db][i] * inv);
  }
}

template <int NB>
int launch_mfma(const AttnArgs& a, int n_tiles, size_t smem, hipStream_t stream) {
  auto kern = latent_attn_mfma_kernel<NB>;
  if (smem > 64 * 1024) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)smem) != hipSuccess)
      return 3;
  }
  hipLaunchKernelGGL(kern, dim3(n_tiles, a.num_splits, (a.H + a.hwin - 1) / a.hwin), dim3(kThreads), smem, stream, a);
  return 0;
}

template <typename CT, int CPL, int PW>
int launch_one(const AttnArgs& a, int n_tiles, size_t smem, hipStream_t stream) {
  auto kern = latent_attn_kernel<CT, CT, CPL, PW>;
  if (smem > 64 * 1024) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)smem) != hipSuccess)
      return 3;
  }
  hipLaunchKernelGGL(kern, dim3(n_tiles, a.num_splits, (a.H + a.hwin - 1) / a.hwin), dim3(kThreads), smem, stream, a);
  return 0;
}

}  // namespace

static int lds_stride(int Dk, size_t esz) {
  // LDS row stride: an odd number of 4-byte words, so lane = key reads hit 64 different banks
  int words = (int)((Dk * esz + 3) / 4);
  if (!(words & 1)) words += 1;
  return (int)(words * 4 / esz);
}

static size_t lds_bytes(int Dk, size_t esz, int PW, int kt) {
  return (size_t)kt * lds_stride(Dk, esz) * esz + (size_t)kWaves * PW * Dk * 4 + (size_t)kWaves * PW * KT * 4;
}

// (row, head) pairs per wave and keys per staged tile of the plain kernel: 8 pairs and 64 keys
// when the tile, the queries and the weights fit the 160 KB of LDS, else fewer keys, then fewer
// pairs; 0: the row is too wide for this kernel
static int pairs_per_wave(int Dk, bool bf, int* kt_out = nullptr) {
  const size_t esz = bf ? 2 : 4, cap = 160 * 1024;
  const int cand[5][2] = {{8, 64}, {8, 32}, {2, 64}, {2, 32}, {2, 16}};
  for (auto& pk : cand)
    if (lds_bytes(Dk, esz, pk[0], pk[1]) <= cap) {
      if (kt_out) *kt_out = pk[1];
      return pk[0];
    }
  return 0;
}

static size_t mfma_lds_bytes(int C, int R) {
  return (size_t)KT * ((C + R) * 2 + 16) + (size_t)C * kVRow + 64 * kVRow + 2 * 64 * sizeof(float);
}

// the matrix-core kernel takes bf16 rows whose latent is a multiple of 64 (1, 2, 3, 4, 6 or 8
// times) and whose rotary part is a multiple of 16 up to 64; ROUNDTABLE_LATENT_FMA=1 pins the
// plain kernel (A/B)
static bool use_mfma(int C, int R, bool bf) {
  static const bool off = [] { const char* e = getenv("ROUNDTABLE_LATENT_FMA"); return e && e[0] == '1'; }();
  const int nb = C / 64;
  return bf && !off && C % 64 == 0 && (nb == 1 || nb == 2 || nb == 3 || nb == 4 || nb == 6 || nb == 8) &&
         R % 16 == 0 && R <= 64 && mfma_lds_bytes(C, R) <= 160 * 1024;
}

// query rows per workgroup: all heads of a row (up to the workgroup's pairs) share the key tile
int latent_rows_per_tile(int H, int C, int R, bool bf) {
  if (use_mfma(C, R, bf)) return H >= 64 ? 1 : 64 / H;
  const int pairs = kWaves * pairs_per_wave(C + R, bf);
  if (pairs == 0) return 0;
  return H >= pairs ? 1 : pairs / H;
}

// 0 ok; 1: `rows` is not latent_rows_per_tile; 2: C too wide; 3: the rows do not fit the LDS
int launch_latent_attention(void* out, const void* q_lat, const void* q, const void* cache, const int* block_tables,
                            const int* cu_q, const int* start_pos, const int* tiles, int n_tiles, const float* sink,
                            float* part_o, float* part_ml, int T, int H, int C, int R, int Dq, int rot_off, int BS,
                            int max_blocks, int rows, int num_splits, float scale, float rot_base, int rot_dims,
                            bool bf, hipStream_t stream) {
  if (n_tiles <= 0 || T <= 0) return 0;
  if (C > 512) return 2;
  const int Dk = C + R;
  const bool mfma = use_mfma(C, R, bf);
  int kt = KT;
  const int PW = mfma ? 16 : pairs_per_wave(Dk, bf, &kt);
  if (PW == 0) return 3;
  const int pairs = kWaves * PW;
  AttnArgs a;
  a.out = out; a.q_lat = q_lat; a.q = q; a.cache = cache; a.block_tables = block_tables; a.cu_q = cu_q;
  a.start_pos = start_pos; a.tiles = tiles; a.sink = sink; a.part_o = part_o; a.part_ml = part_ml;
  a.T = T; a.H = H; a.C = C; a.R = R; a.Dq = Dq; a.rot_off = rot_off; a.BS = BS; a.max_blocks = max_blocks;
  a.rows = rows; a.num_splits = num_splits; a.rot_dims = rot_dims; a.scale = scale;
  a.rot_k = rot_dims > 0 ? (float)(-2.0 * log2((double)rot_base) / rot_dims) : 0.f;
  a.hwin = H < pairs ? H : pairs;
  a.kt = kt;
  if (rows < 1 || rows * a.hwin > pairs) return 1;
  const size_t esz = bf ? 2 : 4;
  a.kstride = lds_stride(Dk, esz);
  const size_t smem = mfma ? 0 : lds_bytes(Dk, esz, PW, kt);
  int rc = 0;
  if (mfma) {
    const size_t sm = mfma_lds_bytes(C, R);
    switch (C / 64) {
      case 1: rc = launch_mfma<1>(a, n_tiles, sm, stream); break;
      case 2: rc = launch_mfma<2>(a, n_tiles, sm, stream); break;
      case 3: rc = launch_mfma<3>(a, n_tiles, sm, stream); break;
      case 4: rc = launch_mfma<4>(a, n_tiles, sm, stream); break;
      case 6: rc = launch_mfma<6>(a, n_tiles, sm, stream); break;
      default: rc = launch_mfma<8>(a, n_tiles, sm, stream); break;
    }
  } else {
#define RT_ATTN(CPLv)                                                                              \
  rc = bf ? (PW == 8 ? launch_one<uint16_t, CPLv, 8>(a, n_tiles, smem, stream)                     \
                     : launch_one<uint16_t, CPLv, 2>(a, n_tiles, smem, stream))                    \
          : (PW == 8 ? launch_one<float, CPLv, 8>(a, n_tiles, smem, stream)                        \
                     : launch_one<float, CPLv, 2>(a, n_tiles, smem, stream))
  if (C <= 64) RT_ATTN(1);
  else if (C <= 128) RT_ATTN(2);
  else if (C <= 256) RT_ATTN(4);
  else RT_ATTN(8);
#undef RT_ATTN
  }
  if (rc == 0 && num_splits > 1) {
    if (bf) hipLaunchKernelGGL((latent_combine_kernel<uint16_t>), dim3(T, H), dim3(C >= 256 ? 256 : 64), 0, stream, (uint16_t*)out, part_o, part_ml, sink, T, H, C, num_splits);
    else hipLaunchKernelGGL((latent_combine_kernel<float>), dim3(T, H), dim3(C >= 256 ? 256 : 64), 0, stream, (float*)out, part_o, part_ml, sink, T, H, C, num_splits);
  }
  return rc;
}
