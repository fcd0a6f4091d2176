// Muon's elementwise stages for gfx950: momentum + Nesterov look-ahead written
// straight into the packed Newton-Schulz batch, and the master update fused with the
// bf16 refresh. Replaces `_muon_mom`, `_muon_mom_t`, `_e_muon_mom`, `_muon_update`,
// `_muon_update_cast`, `_muon_update_cast_t`, `_e_muon_update`, `_transpose_mat`
// (ancora/kernels/muon_ns.py:177-242, 409-427) and `_transpose_e`
// (ancora/kernels/moe.py:370-377). Numpy form: ancora/optim/muon.py:303-309.
//
// Work unit: 4096 elements per block of 256 lanes. A weight that keeps its
// orientation is walked flat, 16 bytes per lane per fp32 access, exactly like AdamW.
// A tall weight (K > N) crosses a 64x64 tile through LDS so that both the (K,N) side
// and the transposed (N,K) side are accessed in 256-byte (fp32) row segments.
#include "common.h"

namespace {

constexpr int kThreads = 256;
constexpr int kBlockElems = 4096;
constexpr int kTile = 64;

constexpr int kPair = 2;     // internal u type: bf16 pair (hi at u, lo at u_lo), see k_mom_multi_pair

struct MomArgs {
  float *buf;
  const void *g;
  void *u;
  int K, N;
  void *u_lo;        // kPair only
  double *fro;       // kPair only: this block's sum of u*u
};
struct UpdArgs {
  float *p32;
  uint16_t *p16;      // may be null
  const void *O;
  int K, N;
  float lr_scale;
  uint32_t seed;
};

__device__ __forceinline__ bool load_ctl(const anc_step_ctl_t *ctl, float &clip) {
  clip = 1.0f;
  if (ctl == nullptr) return true;
  if (ctl->skip != 0u) return false;
  clip = ctl->clip_scale;
  return true;
}

template <int GD>
__device__ __forceinline__ anc_f32x4 load4(const void *p, int64_t e) {
  if (GD == ANC_BF16) {
    const anc_u32x2 b = anc_ld_stream((const anc_u32x2 *)((const uint16_t *)p + e));
    anc_f32x4 r = {__uint_as_float(b.x << 16), __uint_as_float(b.x & 0xFFFF0000u),
                   __uint_as_float(b.y << 16), __uint_as_float(b.y & 0xFFFF0000u)};
    return r;
  }
  return anc_ld_stream((const anc_f32x4 *)((const float *)p + e));
}
template <int UD>
__device__ __forceinline__ void store4(void *p, int64_t e, const float x[4]) {
  if (UD == ANC_BF16 || UD == kPair) {
    const uint32_t b0 = anc_bf16_rne_bits(x[0]), b1 = anc_bf16_rne_bits(x[1]);
    const uint32_t b2 = anc_bf16_rne_bits(x[2]), b3 = anc_bf16_rne_bits(x[3]);
    anc_u32x2 o = {(b0 & 0xFFFFu) | (b1 << 16), (b2 & 0xFFFFu) | (b3 << 16)};
    anc_st_stream((anc_u32x2 *)((uint16_t *)p + e), o);
  } else {
    anc_f32x4 o = {x[0], x[1], x[2], x[3]};
    anc_st_stream((anc_f32x4 *)((float *)p + e), o);
  }
}

// The bf16 pair of x: hi = bf16(x) to `hi`, lo = bf16(x - hi) to `lo`.
__device__ __forceinline__ void store4_pair(void *hi, void *lo, int64_t e, const float x[4]) {
  store4<kPair>(hi, e, x);
  float r[4];
#pragma unroll
  for (int k = 0; k < 4; ++k) r[k] = x[k] - anc_bf16_bits_to_f32(anc_bf16_rne_bits(x[k]));
  store4<kPair>(lo, e, r);
}

// Sum over the block of each lane's `v`, fixed order: xor butterfly inside a wavefront, then
// the 4 wavefront sums left to right. Lane 0 writes the result.
__device__ __forceinline__ void block_sum_to(double v, double *out) {
  __shared__ double wsum[4];
  v = anc_wave_sum_f64(v);
  if ((threadIdx.x & 63) == 0) wsum[threadIdx.x >> 6] = v;
  __syncthreads();
  if (threadIdx.x == 0) *out = ((wsum[0] + wsum[1]) + wsum[2]) + wsum[3];
}

// buf = mom*buf + g';  u = nesterov ? g' + mom*buf : buf     (g' = g*clip)
__device__ __forceinline__ float mom_elem(float g, float &buf, float mom, int nesterov,
                                          float clip) {
  const float gs = g * clip;
  buf = mom * buf + gs;
  return nesterov ? gs + mom * buf : buf;
}

// ---- momentum, orientation kept: flat walk -------------------------------------
template <int GD, int UD>
__device__ __forceinline__ void mom_flat(const MomArgs &a, int64_t blk, float mom, int nesterov,
                                         float clip) {
  const int64_t base = blk * kBlockElems + (int64_t)threadIdx.x * 4;
  anc_f32x4 g4[4], b4[4];
  double ss = 0.0;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int64_t e = base + j * 1024;
    g4[j] = load4<GD>(a.g, e);
    b4[j] = anc_ld_stream((const anc_f32x4 *)(a.buf + e));
  }
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int64_t e = base + j * 1024;
    float gg[4] = {g4[j].x, g4[j].y, g4[j].z, g4[j].w};
    float bb[4] = {b4[j].x, b4[j].y, b4[j].z, b4[j].w};
    float uu[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) uu[k] = mom_elem(gg[k], bb[k], mom, nesterov, clip);
    anc_f32x4 bo = {bb[0], bb[1], bb[2], bb[3]};
    anc_st_stream((anc_f32x4 *)(a.buf + e), bo);
    if (UD == kPair) {
      store4_pair(a.u, a.u_lo, e, uu);
#pragma unroll
      for (int k = 0; k < 4; ++k) ss += (double)uu[k] * (double)uu[k];
    } else {
      store4<UD>(a.u, e, uu);
    }
  }
  if (UD == kPair) block_sum_to(ss, a.fro);
}

// ---- momentum, transposed store: 64x64 tile through LDS ------------------------
template <int GD, int UD>
__device__ __forceinline__ void mom_tile_t(const MomArgs &a, int64_t tile, float mom,
                                           int nesterov, float clip) {
  __shared__ float lds[kTile][kTile + 1];
  const int tiles_n = a.N / kTile;
  const int tr = (int)(tile / tiles_n), tc = (int)(tile % tiles_n);
  const int c4 = (threadIdx.x & 15) * 4, r0 = threadIdx.x >> 4;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = r0 + 16 * i;
    const int64_t e = (int64_t)(tr * kTile + r) * a.N + tc * kTile + c4;
    const anc_f32x4 g = load4<GD>(a.g, e);
    const anc_f32x4 b = anc_ld_stream((const anc_f32x4 *)(a.buf + e));
    float gg[4] = {g.x, g.y, g.z, g.w};
    float bb[4] = {b.x, b.y, b.z, b.w};
#pragma unroll
    for (int k = 0; k < 4; ++k) lds[r][c4 + k] = mom_elem(gg[k], bb[k], mom, nesterov, clip);
    anc_f32x4 bo = {bb[0], bb[1], bb[2], bb[3]};
    anc_st_stream((anc_f32x4 *)(a.buf + e), bo);
  }
  __syncthreads();
  // u^T is (N,K): row tc*64 + r, columns tr*64 + c4 ..
  double ss = 0.0;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = r0 + 16 * i;
    float uu[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) uu[k] = lds[c4 + k][r];
    const int64_t e = (int64_t)(tc * kTile + r) * a.K + tr * kTile + c4;
    if (UD == kPair) {
      store4_pair(a.u, a.u_lo, e, uu);
#pragma unroll
      for (int k = 0; k < 4; ++k) ss += (double)uu[k] * (double)uu[k];
    } else {
      store4<UD>(a.u, e, uu);
    }
  }
  if (UD == kPair) block_sum_to(ss, a.fro);
}

// ---- update: p32 -= lr_scale*O; p16 = bf16(p32) ----------------------------------
template <int SR>
__device__ __forceinline__ void upd_store(const UpdArgs &a, int64_t e, const float o[4],
                                          const anc_f32x4 &p, uint32_t (&hb)[4]) {
  float pp[4] = {p.x, p.y, p.z, p.w};
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    pp[k] = pp[k] - a.lr_scale * o[k];
    const uint64_t i = (uint64_t)(e + k);
    hb[k] = SR ? anc_bf16_sr_bits(pp[k], (uint32_t)(i >> 6), (uint32_t)(i & 63u), a.seed)
               : anc_bf16_rne_bits(pp[k]);
  }
  anc_f32x4 po = {pp[0], pp[1], pp[2], pp[3]};
  anc_st_stream((anc_f32x4 *)(a.p32 + e), po);
  if (a.p16 != nullptr) {
    anc_u32x2 ho = {(hb[0] & 0xFFFFu) | (hb[1] << 16), (hb[2] & 0xFFFFu) | (hb[3] << 16)};
    anc_st_stream((anc_u32x2 *)(a.p16 + e), ho);
  }
}

template <int SR>
__device__ __forceinline__ void upd_store(const UpdArgs &a, int64_t e, const float o[4],
                                          const anc_f32x4 &p) {
  uint32_t hb[4];
  upd_store<SR>(a, e, o, p, hb);
}

template <int OD, int SR>
__device__ __forceinline__ void upd_flat(const UpdArgs &a, int64_t blk) {
  const int64_t base = blk * kBlockElems + (int64_t)threadIdx.x * 4;
  anc_f32x4 o4[4], p4[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int64_t e = base + j * 1024;
    o4[j] = load4<OD>(a.O, e);
    p4[j] = anc_ld_stream((const anc_f32x4 *)(a.p32 + e));
  }
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const float oo[4] = {o4[j].x, o4[j].y, o4[j].z, o4[j].w};
    upd_store<SR>(a, base + j * 1024, oo, p4[j]);
  }
}

// ---- update that also refreshes a transposed bf16 copy of the weight -------------------
// p16t is (N,K): the copy the MoE backward reads (ancora/kernels/moe.py:370-377, 593-597 runs a
// separate transpose kernel over p16 after the step). 64x64 tile of W per block in either
// orientation of O; the new bf16 values cross LDS once more and leave as rows of p16t.
template <int OD, int SR>
__device__ __forceinline__ void upd_tile_p16t(const UpdArgs &a, int64_t tile, bool o_transposed,
                                              uint16_t *p16t) {
  __shared__ float ldsO[kTile][kTile + 1];
  __shared__ uint16_t ldsH[kTile][kTile + 2];
  const int tiles_n = a.N / kTile;
  const int tr = (int)(tile / tiles_n), tc = (int)(tile % tiles_n);
  const int c4 = (threadIdx.x & 15) * 4, r0 = threadIdx.x >> 4;
  if (o_transposed) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int r = r0 + 16 * i;
      const int64_t e = (int64_t)(tc * kTile + r) * a.K + tr * kTile + c4;
      const anc_f32x4 o = load4<OD>(a.O, e);
      ldsO[r][c4] = o.x; ldsO[r][c4 + 1] = o.y; ldsO[r][c4 + 2] = o.z; ldsO[r][c4 + 3] = o.w;
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = r0 + 16 * i;
    const int64_t e = (int64_t)(tr * kTile + r) * a.N + tc * kTile + c4;
    const anc_f32x4 p = anc_ld_stream((const anc_f32x4 *)(a.p32 + e));
    float oo[4];
    if (o_transposed) {
#pragma unroll
      for (int k = 0; k < 4; ++k) oo[k] = ldsO[c4 + k][r];
    } else {
      const anc_f32x4 o = load4<OD>(a.O, e);
      oo[0] = o.x; oo[1] = o.y; oo[2] = o.z; oo[3] = o.w;
    }
    uint32_t hb[4];
    upd_store<SR>(a, e, oo, p, hb);
    if (p16t != nullptr) {
#pragma unroll
      for (int k = 0; k < 4; ++k) ldsH[r][c4 + k] = (uint16_t)hb[k];
    }
  }
  if (p16t == nullptr) return;        // uniform over the block
  __syncthreads();
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = r0 + 16 * i;
    const uint32_t h0 = ldsH[c4][r], h1 = ldsH[c4 + 1][r], h2 = ldsH[c4 + 2][r], h3 = ldsH[c4 + 3][r];
    const anc_u32x2 ho = {h0 | (h1 << 16), h2 | (h3 << 16)};
    anc_st_stream((anc_u32x2 *)(p16t + (int64_t)(tc * kTile + r) * a.K + tr * kTile + c4), ho);
  }
}

template <int OD, int SR>
__device__ __forceinline__ void upd_tile_t(const UpdArgs &a, int64_t tile) {
  upd_tile_p16t<OD, SR>(a, tile, true, nullptr);
}

// ---- kernels -----------------------------------------------------------------------
template <int GD, int UD, int TR>
__global__ void __launch_bounds__(kThreads)
k_mom(MomArgs a, float mom, int nesterov, const anc_step_ctl_t *__restrict__ ctl) {
  float clip;
  if (!load_ctl(ctl, clip)) return;
  if (TR) mom_tile_t<GD, UD>(a, (int64_t)blockIdx.x, mom, nesterov, clip);
  else    mom_flat<GD, UD>(a, (int64_t)blockIdx.x, mom, nesterov, clip);
}

template <int OD, int SR, int TR>
__global__ void __launch_bounds__(kThreads)
k_upd(UpdArgs a, const anc_step_ctl_t *__restrict__ ctl) {
  float clip;
  if (!load_ctl(ctl, clip)) return;
  if (TR) upd_tile_t<OD, SR>(a, (int64_t)blockIdx.x);
  else    upd_flat<OD, SR>(a, (int64_t)blockIdx.x);
}

__device__ __forceinline__ const anc_muon_desc_t &find_weight(const anc_muon_desc_t *table,
                                                              int n, int64_t blk) {
  int lo = 0, hi = n - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (table[mid].tile0 <= blk) lo = mid; else hi = mid - 1;
  }
  return table[lo];
}

template <int UD>
__global__ void __launch_bounds__(kThreads)
k_mom_multi(const anc_muon_desc_t *__restrict__ table, int n_weights, float mom, int nesterov,
            const anc_step_ctl_t *__restrict__ ctl) {
  float clip;
  if (!load_ctl(ctl, clip)) return;
  const anc_muon_desc_t d = find_weight(table, n_weights, (int64_t)blockIdx.x);
  const int64_t local = (int64_t)blockIdx.x - d.tile0;
  MomArgs a{(float *)d.buf, (const void *)d.g, (void *)d.u, d.K, d.N, nullptr, nullptr};
  if (d.transpose) {
    if (d.g_dtype == ANC_BF16) mom_tile_t<ANC_BF16, UD>(a, local, mom, nesterov, clip);
    else                       mom_tile_t<ANC_F32, UD>(a, local, mom, nesterov, clip);
  } else {
    if (d.g_dtype == ANC_BF16) mom_flat<ANC_BF16, UD>(a, local, mom, nesterov, clip);
    else                       mom_flat<ANC_F32, UD>(a, local, mom, nesterov, clip);
  }
}

// Momentum straight into the Newton-Schulz input format. d.u is the weight's slice of the
// packed batch counted in fp32 elements from `base` (where the chain's fp32 result will land);
// the bf16 pair of u goes to the same element offset in two bf16 arrays, hi at `base`, lo
// `lo_off` bytes further (together the same 4 bytes per element). Block b also leaves the sum
// of its 4096 u*u in fro[b], so that the Frobenius norm needs no further pass over the data:
// a weight's blocks are consecutive, K*N/4096 of them.
__global__ void __launch_bounds__(kThreads)
k_mom_multi_pair(const anc_muon_desc_t *__restrict__ table, int n_weights, float mom, int nesterov,
                 uint64_t base, int64_t lo_off, double *__restrict__ fro,
                 const anc_step_ctl_t *__restrict__ ctl) {
  float clip;
  if (!load_ctl(ctl, clip)) return;
  const anc_muon_desc_t d = find_weight(table, n_weights, (int64_t)blockIdx.x);
  const int64_t local = (int64_t)blockIdx.x - d.tile0;
  const uint64_t hi = base + (d.u - base) / 2;
  MomArgs a{(float *)d.buf, (const void *)d.g, (void *)hi, d.K, d.N, (void *)(hi + (uint64_t)lo_off),
            fro + blockIdx.x};
  if (d.transpose) {
    if (d.g_dtype == ANC_BF16) mom_tile_t<ANC_BF16, kPair>(a, local, mom, nesterov, clip);
    else                       mom_tile_t<ANC_F32, kPair>(a, local, mom, nesterov, clip);
  } else {
    if (d.g_dtype == ANC_BF16) mom_flat<ANC_BF16, kPair>(a, local, mom, nesterov, clip);
    else                       mom_flat<ANC_F32, kPair>(a, local, mom, nesterov, clip);
  }
}

struct LrScales { float v[ANC_MUON_MAX_SCALES]; };

template <int OD, int SR>
__global__ void __launch_bounds__(kThreads)
k_upd_multi(const anc_muon_desc_t *__restrict__ table, int n_weights, LrScales scales,
            uint32_t seed_base, int step_seed, const anc_step_ctl_t *__restrict__ ctl) {
  float clip;
  if (!load_ctl(ctl, clip)) return;
  if (step_seed) seed_base += ANC_SR_SEED_STRIDE * ctl->t;      // steps counted on the device
  const anc_muon_desc_t d = find_weight(table, n_weights, (int64_t)blockIdx.x);
  const int64_t local = (int64_t)blockIdx.x - d.tile0;
  UpdArgs a{(float *)d.p32, (uint16_t *)d.p16, (const void *)d.u, d.K, d.N,
            scales.v[d.scale_idx & (ANC_MUON_MAX_SCALES - 1)], seed_base + d.seed};
  if (d.p16t != 0 || d.transpose)
    upd_tile_p16t<OD, SR>(a, local, d.transpose != 0, (uint16_t *)d.p16t);
  else
    upd_flat<OD, SR>(a, local);
}

// bf16 transpose, batched: XT[e] (N,M) = X[e] (M,N)^T, 64x64 tiles through LDS.
__global__ void __launch_bounds__(kThreads)
k_transpose_bf16(const uint16_t *__restrict__ X, uint16_t *__restrict__ XT, int M, int N) {
  __shared__ uint16_t lds[kTile][kTile + 2];
  const int tiles_n = N / kTile, tiles_m = M / kTile;
  const int64_t per = (int64_t)tiles_m * tiles_n;
  const int64_t e = (int64_t)blockIdx.x / per;
  const int64_t tile = (int64_t)blockIdx.x % per;
  const int tr = (int)(tile / tiles_n), tc = (int)(tile % tiles_n);
  const uint16_t *x = X + e * (int64_t)M * N;
  uint16_t *xt = XT + e * (int64_t)M * N;
  const int c4 = (threadIdx.x & 15) * 4, r0 = threadIdx.x >> 4;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = r0 + 16 * i;
    const anc_u32x2 v = *(const anc_u32x2 *)(x + (int64_t)(tr * kTile + r) * N + tc * kTile + c4);
    lds[r][c4] = (uint16_t)(v.x & 0xFFFFu); lds[r][c4 + 1] = (uint16_t)(v.x >> 16);
    lds[r][c4 + 2] = (uint16_t)(v.y & 0xFFFFu); lds[r][c4 + 3] = (uint16_t)(v.y >> 16);
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = r0 + 16 * i;
    const uint32_t a0 = lds[c4][r], a1 = lds[c4 + 1][r], a2 = lds[c4 + 2][r], a3 = lds[c4 + 3][r];
    anc_u32x2 o = {a0 | (a1 << 16), a2 | (a3 << 16)};
    *(anc_u32x2 *)(xt + (int64_t)(tc * kTile + r) * M + tr * kTile + c4) = o;
  }
}

__global__ void __launch_bounds__(kThreads)
k_bf16_to_f32(const uint16_t *__restrict__ src, float *__restrict__ dst, int64_t n) {
  const int64_t e = ((int64_t)blockIdx.x * kThreads + threadIdx.x) * 4;
  if (e >= n) return;
  const anc_f32x4 v = load4<ANC_BF16>(src, e);
  *(anc_f32x4 *)(dst + e) = v;
}
__global__ void __launch_bounds__(kThreads)
k_f32_to_bf16(const float *__restrict__ src, uint16_t *__restrict__ dst, int64_t n) {
  const int64_t e = ((int64_t)blockIdx.x * kThreads + threadIdx.x) * 4;
  if (e >= n) return;
  const anc_f32x4 v = *(const anc_f32x4 *)(src + e);
  const float x[4] = {v.x, v.y, v.z, v.w};
  store4<ANC_BF16>(dst, e, x);
}

int check_kn(int64_t K, int64_t N, const char *who) {
  ANC_REQUIRE(K > 0 && N > 0 && K % 64 == 0 && N % 64 == 0,
              "%s: (K,N)=(%lld,%lld) must be positive multiples of 64", who, (long long)K,
              (long long)N);
  ANC_REQUIRE(K < (1ll << 30) && N < (1ll << 30) && (K * N) / kBlockElems < (1ll << 31),
              "%s: matrix too large", who);
  return ANC_OK;
}

}  // namespace

extern "C" int anc_muon_momentum(uint64_t buf, uint64_t g, uint64_t u, int64_t K, int64_t N,
                                 float mom, int nesterov, int transpose_out, int g_dtype,
                                 int u_dtype, uint64_t ctl, uint64_t stream) {
  if (int rc = check_kn(K, N, "anc_muon_momentum")) return rc;
  ANC_REQUIRE(buf && g && u, "anc_muon_momentum: null device pointer");
  ANC_REQUIRE((g_dtype == ANC_F32 || g_dtype == ANC_BF16) && (u_dtype == ANC_F32 || u_dtype == ANC_BF16),
              "anc_muon_momentum: bad dtype");
  ANC_REQUIRE(((buf | g | u) & 15) == 0, "anc_muon_momentum: pointers must be 16-byte aligned");
  MomArgs a{(float *)buf, (const void *)g, (void *)u, (int)K, (int)N, nullptr, nullptr};
  const anc_step_ctl_t *c = (const anc_step_ctl_t *)ctl;
  const dim3 grid((unsigned)((K * N) / kBlockElems)), block(kThreads);
  hipStream_t s = anc_stream(stream);
  AncProfScope prof(ANC_PROF_MUON_MOM, s);
#define MOM(GD, UD, TR) hipLaunchKernelGGL((k_mom<GD, UD, TR>), grid, block, 0, s, a, mom, nesterov, c)
  const int sel = (g_dtype == ANC_BF16 ? 4 : 0) | (u_dtype == ANC_BF16 ? 2 : 0) | (transpose_out ? 1 : 0);
  switch (sel) {
    case 0: MOM(ANC_F32, ANC_F32, 0); break;   case 1: MOM(ANC_F32, ANC_F32, 1); break;
    case 2: MOM(ANC_F32, ANC_BF16, 0); break;  case 3: MOM(ANC_F32, ANC_BF16, 1); break;
    case 4: MOM(ANC_BF16, ANC_F32, 0); break;  case 5: MOM(ANC_BF16, ANC_F32, 1); break;
    case 6: MOM(ANC_BF16, ANC_BF16, 0); break; default: MOM(ANC_BF16, ANC_BF16, 1); break;
  }
#undef MOM
  ANC_LAUNCH_CHECK();
  return ANC_OK;
}

extern "C" int anc_muon_update(uint64_t p32, uint64_t p16, uint64_t O, int64_t K, int64_t N,
                               float lr_scale, int transpose_in, int o_dtype, int sr,
                               uint32_t seed, uint64_t ctl, uint64_t stream) {
  if (int rc = check_kn(K, N, "anc_muon_update")) return rc;
  ANC_REQUIRE(p32 && O, "anc_muon_update: null device pointer");
  ANC_REQUIRE(o_dtype == ANC_F32 || o_dtype == ANC_BF16, "anc_muon_update: bad dtype");
  ANC_REQUIRE(((p32 | O) & 15) == 0 && (p16 & 7) == 0, "anc_muon_update: misaligned pointers");
  ANC_REQUIRE(sr == 0 || sr == ANC_SR_ON, "anc_muon_update: sr must be 0 or ANC_SR_ON");
  UpdArgs a{(float *)p32, (uint16_t *)p16, (const void *)O, (int)K, (int)N, lr_scale, seed};
  const anc_step_ctl_t *c = (const anc_step_ctl_t *)ctl;
  const dim3 grid((unsigned)((K * N) / kBlockElems)), block(kThreads);
  hipStream_t s = anc_stream(stream);
  AncProfScope prof(ANC_PROF_MUON_UPD, s);
#define UPD(OD, SR, TR) hipLaunchKernelGGL((k_upd<OD, SR, TR>), grid, block, 0, s, a, c)
  const int sel = (o_dtype == ANC_BF16 ? 4 : 0) | (sr ? 2 : 0) | (transpose_in ? 1 : 0);
  switch (sel) {
    case 0: UPD(ANC_F32, 0, 0); break;   case 1: UPD(ANC_F32, 0, 1); break;
    case 2: UPD(ANC_F32, 1, 0); break;   case 3: UPD(ANC_F32, 1, 1); break;
    case 4: UPD(ANC_BF16, 0, 0); break;  case 5: UPD(ANC_BF16, 0, 1); break;
    case 6: UPD(ANC_BF16, 1, 0); break;  default: UPD(ANC_BF16, 1, 1); break;
  }
#undef UPD
  ANC_LAUNCH_CHECK();
  return ANC_OK;
}

extern "C" int anc_muon_momentum_multi(uint64_t desc_table, int32_t n_weights, int64_t total_tiles,
                                       float mom, int nesterov, int u_dtype, uint64_t ctl,
                                       uint64_t stream) {
  ANC_REQUIRE(desc_table != 0 && n_weights > 0, "anc_muon_momentum_multi: empty descriptor table");
  ANC_REQUIRE(total_tiles > 0 && total_tiles < (1ll << 31), "anc_muon_momentum_multi: bad total_tiles");
  ANC_REQUIRE(u_dtype == ANC_F32 || u_dtype == ANC_BF16, "anc_muon_momentum_multi: bad dtype");
  const anc_muon_desc_t *tab = (const anc_muon_desc_t *)desc_table;
  const anc_step_ctl_t *c = (const anc_step_ctl_t *)ctl;
  const dim3 grid((unsigned)total_tiles), block(kThreads);
  AncProfScope prof(ANC_PROF_MUON_MOM, anc_stream(stream));
  if (u_dtype == ANC_BF16)
    hipLaunchKernelGGL(k_mom_multi<ANC_BF16>, grid, block, 0, anc_stream(stream), tab, (int)n_weights,
                       mom, nesterov, c);
  else
    hipLaunchKernelGGL(k_mom_multi<ANC_F32>, grid, block, 0, anc_stream(stream), tab, (int)n_weights,
                       mom, nesterov, c);
  ANC_LAUNCH_CHECK();
  return ANC_OK;
}

extern "C" int anc_muon_momentum_multi_pair(uint64_t desc_table, int32_t n_weights, int64_t total_tiles,
                                            float mom, int nesterov, uint64_t pair_base,
                                            int64_t lo_offset_bytes, uint64_t fro_partials,
                                            uint64_t ctl, uint64_t stream) {
  ANC_REQUIRE(desc_table != 0 && n_weights > 0, "anc_muon_momentum_multi_pair: empty descriptor table");
  ANC_REQUIRE(total_tiles > 0 && total_tiles < (1ll << 31), "anc_muon_momentum_multi_pair: bad total_tiles");
  ANC_REQUIRE(pair_base != 0 && (pair_base & 15) == 0 && lo_offset_bytes > 0 && (lo_offset_bytes & 15) == 0,
              "anc_muon_momentum_multi_pair: pair buffer must be 16-byte aligned");
  ANC_REQUIRE(fro_partials != 0 && (fro_partials & 7) == 0, "anc_muon_momentum_multi_pair: null partials");
  AncProfScope prof(ANC_PROF_MUON_MOM, anc_stream(stream));
  hipLaunchKernelGGL(k_mom_multi_pair, dim3((unsigned)total_tiles), dim3(kThreads), 0, anc_stream(stream),
                     (const anc_muon_desc_t *)desc_table, (int)n_weights, mom, nesterov, pair_base,
                     lo_offset_bytes, (double *)fro_partials, (const anc_step_ctl_t *)ctl);
  ANC_LAUNCH_CHECK();
  return ANC_OK;
}

extern "C" int anc_muon_update_multi(uint64_t desc_table, int32_t n_weights, int64_t total_tiles,
                                     const float *lr_scales, int o_dtype, int sr,
                                     uint32_t seed_base, uint64_t ctl, uint64_t stream) {
  ANC_REQUIRE(desc_table != 0 && n_weights > 0, "anc_muon_update_multi: empty descriptor table");
  ANC_REQUIRE(lr_scales != nullptr, "anc_muon_update_multi: null lr_scales");
  LrScales sc;
  for (int i = 0; i < ANC_MUON_MAX_SCALES; ++i) sc.v[i] = lr_scales[i];
  ANC_REQUIRE(total_tiles > 0 && total_tiles < (1ll << 31), "anc_muon_update_multi: bad total_tiles");
  ANC_REQUIRE(o_dtype == ANC_F32 || o_dtype == ANC_BF16, "anc_muon_update_multi: bad dtype");
  const anc_muon_desc_t *tab = (const anc_muon_desc_t *)desc_table;
  const anc_step_ctl_t *c = (const anc_step_ctl_t *)ctl;
  const dim3 grid((unsigned)total_tiles), block(kThreads);
  hipStream_t s = anc_stream(stream);
  AncProfScope prof(ANC_PROF_MUON_UPD, s);
  const int step_seed = (sr & ANC_SR_STEP_SEED) ? 1 : 0;
  ANC_REQUIRE(!step_seed || ctl != 0, "anc_muon_update_multi: ANC_SR_STEP_SEED needs the control block");
  const int sel = (o_dtype == ANC_BF16 ? 2 : 0) | (sr ? 1 : 0);
  switch (sel) {
    case 0: hipLaunchKernelGGL((k_upd_multi<ANC_F32, 0>), grid, block, 0, s, tab, (int)n_weights, sc, seed_base, step_seed, c); break;
    case 1: hipLaunchKernelGGL((k_upd_multi<ANC_F32, 1>), grid, block, 0, s, tab, (int)n_weights, sc, seed_base, step_seed, c); break;
    case 2: hipLaunchKernelGGL((k_upd_multi<ANC_BF16, 0>), grid, block, 0, s, tab, (int)n_weights, sc, seed_base, step_seed, c); break;
    default: hipLaunchKernelGGL((k_upd_multi<ANC_BF16, 1>), grid, block, 0, s, tab, (int)n_weights, sc, seed_base, step_seed, c); break;
  }
  ANC_LAUNCH_CHECK();
  return ANC_OK;
}

extern "C" int anc_transpose_bf16(uint64_t X, uint64_t XT, int64_t E, int64_t M, int64_t N,
                                  uint64_t stream) {
  if (int rc = check_kn(M, N, "anc_transpose_bf16")) return rc;
  ANC_REQUIRE(X && XT && X != XT && E > 0, "anc_transpose_bf16: bad arguments");
  ANC_REQUIRE(((X | XT) & 7) == 0, "anc_transpose_bf16: pointers must be 8-byte aligned");
  const int64_t blocks = E * (M / kTile) * (N / kTile);
  ANC_REQUIRE(blocks < (1ll << 31), "anc_transpose_bf16: batch too large");
  AncProfScope prof(ANC_PROF_MISC, anc_stream(stream));
  hipLaunchKernelGGL(k_transpose_bf16, dim3((unsigned)blocks), dim3(kThreads), 0, anc_stream(stream),
                     (const uint16_t *)X, (uint16_t *)XT, (int)M, (int)N);
  ANC_LAUNCH_CHECK();
  return ANC_OK;
}

extern "C" int anc_bf16_to_f32(uint64_t src, uint64_t dst, int64_t n, uint64_t stream) {
  ANC_REQUIRE(src && dst && n > 0 && n % 4 == 0 && (src & 7) == 0 && (dst & 15) == 0,
              "anc_bf16_to_f32: bad arguments");
  const int64_t blocks = (n / 4 + kThreads - 1) / kThreads;
  ANC_REQUIRE(blocks < (1ll << 31), "anc_bf16_to_f32: too large");
  AncProfScope prof(ANC_PROF_MISC, anc_stream(stream));
  hipLaunchKernelGGL(k_bf16_to_f32, dim3((unsigned)blocks), dim3(kThreads), 0, anc_stream(stream),
                     (const uint16_t *)src, (float *)dst, n);
  ANC_LAUNCH_CHECK();
  return ANC_OK;
}
extern "C" int anc_f32_to_bf16(uint64_t src, uint64_t dst, int64_t n, uint64_t stream) {
  ANC_REQUIRE(src && dst && n > 0 && n % 4 == 0 && (src & 15) == 0 && (dst & 7) == 0,
              "anc_f32_to_bf16: bad arguments");
  const int64_t blocks = (n / 4 + kThreads - 1) / kThreads;
  ANC_REQUIRE(blocks < (1ll << 31), "anc_f32_to_bf16: too large");
  AncProfScope prof(ANC_PROF_MISC, anc_stream(stream));
  hipLaunchKernelGGL(k_f32_to_bf16, dim3((unsigned)blocks), dim3(kThreads), 0, anc_stream(stream),
                     (const float *)src, (uint16_t *)dst, n);
  ANC_LAUNCH_CHECK();
  return ANC_OK;
}
