// Single-pass fused AdamW for gfx950: fp32 master weights and m/v state, bias
// correction, decoupled weight decay, global-clip scaling, skip-step guard and the
// bf16 downcast (RNE or counter-based stochastic rounding) in one sweep over HBM.
// Replaces the `_adamw` cuda-tile kernel (ancora/optim/adamw.py:23-41) and the bf16
// refresh `_cast_bf16` (ancora/kernels/fused.py:285-290).
//
// Data layout: every tensor is a flat run of n elements (n % 64 == 0, the reference's
// (numel/64, 64) view, ancora/optim/adamw.py:20,79). A block of 256 lanes owns 4096
// consecutive elements and walks them as four 1024-element slabs; in a slab lane t
// owns elements [4t, 4t+4): one 16-byte access per fp32 stream (a wavefront covers
// 1 KiB contiguous) and one 8-byte access per bf16 stream. All sixteen loads of a
// lane are issued before the arithmetic starts.
//
// Arithmetic: compiled with -ffp-contract=off; divide and sqrt are the correctly
// rounded forms, so each element reproduces the numpy fp32 evaluation of
// tests/optim/test_adamw.py:37-41 bit for bit.
#include "common.h"

namespace {

#ifndef ADAMW_UNROLL
#define ADAMW_UNROLL 4
#endif
#ifndef ADAMW_LD_NT
#define ADAMW_LD_NT 1
#endif
#ifndef ADAMW_ST_NT
#define ADAMW_ST_NT 1
#endif
constexpr int kThreads = 256;
constexpr int kVec = 4;
constexpr int kUnroll = ADAMW_UNROLL;
template <typename T> __device__ __forceinline__ T ld_(const T *p) {
  return ADAMW_LD_NT ? __builtin_nontemporal_load(p) : *p;
}
template <typename T> __device__ __forceinline__ void st_(T *p, T v) {
  if (ADAMW_ST_NT) __builtin_nontemporal_store(v, p); else *p = v;
}
constexpr int kSlab = kThreads * kVec;          // 1024 elements
constexpr int kBlockElems = kSlab * kUnroll;    // 4096 elements

struct Tensor {
  const void *g;
  float *m, *v, *p32;
  uint16_t *p16;
  int64_t n;
  float wd;
  uint32_t seed;
};

template <int FORM>
__device__ __forceinline__ void adamw_elem(float g, float &m, float &v, float &p,
                                           const anc_adamw_hyper_t &h, float wd, float clip) {
  const float gs = g * clip;
  if (FORM == ANC_ADAMW_FORM_DIV) {
    m = h.beta1 * m + h.omb1 * gs;
    v = h.beta2 * v + (h.omb2 * gs) * gs;
    const float mh = m / h.bc1;
    const float vh = v / h.bc2;
    p = p - h.lr * (mh / (sqrtf(vh) + h.eps) + wd * p);
  } else {
    const float o1 = 1.0f - h.beta1, o2 = 1.0f - h.beta2;
    m = h.beta1 * m + o1 * gs;
    v = h.beta2 * v + (o2 * gs) * gs;
    p = p - h.lr * ((m * h.bc1) / (sqrtf(v * h.bc2) + h.eps) + wd * p);
  }
}

template <int GD, int FORM, int SR>
__device__ __forceinline__ void adamw_block(const Tensor &t, int64_t blk,
                                            const anc_adamw_hyper_t &h, float clip) {
  const int64_t base = blk * kBlockElems + (int64_t)threadIdx.x * kVec;
  anc_f32x4 g4[kUnroll], m4[kUnroll], v4[kUnroll], p4[kUnroll];
  bool live[kUnroll];
#pragma unroll
  for (int j = 0; j < kUnroll; ++j) {
    const int64_t e = base + (int64_t)j * kSlab;
    live[j] = e < t.n;
    if (live[j]) {
      if (GD == ANC_BF16) {
        const anc_u32x2 gb = ld_((const anc_u32x2 *)((const uint16_t *)t.g + e));
        g4[j].x = __uint_as_float(gb.x << 16);
        g4[j].y = __uint_as_float(gb.x & 0xFFFF0000u);
        g4[j].z = __uint_as_float(gb.y << 16);
        g4[j].w = __uint_as_float(gb.y & 0xFFFF0000u);
      } else {
        g4[j] = ld_((const anc_f32x4 *)((const float *)t.g + e));
      }
      m4[j] = ld_((const anc_f32x4 *)(t.m + e));
      v4[j] = ld_((const anc_f32x4 *)(t.v + e));
      p4[j] = ld_((const anc_f32x4 *)(t.p32 + e));
    }
  }
#pragma unroll
  for (int j = 0; j < kUnroll; ++j) {
    if (!live[j]) continue;
    const int64_t e = base + (int64_t)j * kSlab;
    float gg[4] = {g4[j].x, g4[j].y, g4[j].z, g4[j].w};
    float mm[4] = {m4[j].x, m4[j].y, m4[j].z, m4[j].w};
    float vv[4] = {v4[j].x, v4[j].y, v4[j].z, v4[j].w};
    float pp[4] = {p4[j].x, p4[j].y, p4[j].z, p4[j].w};
    uint32_t hb[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      adamw_elem<FORM>(gg[k], mm[k], vv[k], pp[k], h, t.wd, clip);
      if (SR) {
        const uint64_t i = (uint64_t)(e + k);
        hb[k] = anc_bf16_sr_bits(pp[k], (uint32_t)(i >> 6), (uint32_t)(i & 63u), t.seed);
      } else {
        hb[k] = anc_bf16_rne_bits(pp[k]);
      }
    }
    anc_f32x4 mo = {mm[0], mm[1], mm[2], mm[3]};
    anc_f32x4 vo = {vv[0], vv[1], vv[2], vv[3]};
    anc_f32x4 po = {pp[0], pp[1], pp[2], pp[3]};
    anc_u32x2 ho = {(hb[0] & 0xFFFFu) | (hb[1] << 16), (hb[2] & 0xFFFFu) | (hb[3] << 16)};
    st_((anc_f32x4 *)(t.m + e), mo);
    st_((anc_f32x4 *)(t.v + e), vo);
    st_((anc_f32x4 *)(t.p32 + e), po);
    st_((anc_u32x2 *)(t.p16 + e), ho);
  }
}

__device__ __forceinline__ bool load_ctl(const anc_step_ctl_t *ctl, float &clip) {
  clip = 1.0f;
  if (ctl == nullptr) return true;
  if (ctl->skip != 0u) return false;
  clip = ctl->clip_scale;
  return true;
}

struct RowStep { float bc1, bc2, lr; uint32_t seed_base; };   // anc_adamw_step_t; entry s: counted step s (1-based)

// Steps counted on the device: the bias corrections of step ctl->t from the table the host filled
// ahead (the same fp32 values it would pass per step), the rounding seed from the count itself.
__device__ __forceinline__ void step_scalars(anc_adamw_hyper_t &h, const anc_step_ctl_t *ctl) {
  if (ctl == nullptr) return;
  const uint32_t t = ctl->t;
  if (h.step_table != 0) {
    const uint32_t i = t < 1u ? 1u : (t > (uint32_t)h.step_cap ? (uint32_t)h.step_cap : t);
    const RowStep rs = ((const RowStep *)h.step_table)[i];
    h.bc1 = rs.bc1;
    h.bc2 = rs.bc2;
  }
  if (h.sr & ANC_SR_STEP_SEED) h.seed_base += ANC_SR_SEED_STRIDE * t;
}

template <int GD, int FORM, int SR>
__global__ void __launch_bounds__(kThreads)
k_adamw(Tensor t, anc_adamw_hyper_t h, const anc_step_ctl_t *__restrict__ ctl) {
  float clip;
  if (!load_ctl(ctl, clip)) return;
  const uint32_t seed0 = h.seed_base;
  step_scalars(h, ctl);
  t.seed += h.seed_base - seed0;
  adamw_block<GD, FORM, SR>(t, (int64_t)blockIdx.x, h, clip);
}

template <int FORM, int SR>
__global__ void __launch_bounds__(kThreads)
k_adamw_multi(const anc_adamw_desc_t *__restrict__ table, int n_tensors, anc_adamw_hyper_t h,
              const anc_step_ctl_t *__restrict__ ctl) {
  float clip;
  if (!load_ctl(ctl, clip)) return;
  step_scalars(h, ctl);
  const int64_t blk = (int64_t)blockIdx.x;
  // Last tensor whose first block is <= blk (the table is sorted by blk0).
  int lo = 0, hi = n_tensors - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (table[mid].blk0 <= blk) lo = mid; else hi = mid - 1;
  }
  const anc_adamw_desc_t d = table[lo];
  Tensor t;
  t.g = (const void *)d.g;
  t.m = (float *)d.m;
  t.v = (float *)d.v;
  t.p32 = (float *)d.p32;
  t.p16 = (uint16_t *)d.p16;
  t.n = d.n;
  t.wd = d.wd;
  t.seed = h.seed_base + d.seed;
  if (d.g_dtype == ANC_BF16)
    adamw_block<ANC_BF16, FORM, SR>(t, blk - d.blk0, h, clip);
  else
    adamw_block<ANC_F32, FORM, SR>(t, blk - d.blk0, h, clip);
}

template <int SR>
__global__ void __launch_bounds__(kThreads)
k_cast_bf16(const float *__restrict__ p32, uint16_t *__restrict__ p16, int64_t n, uint32_t seed) {
  const int64_t base = (int64_t)blockIdx.x * kBlockElems + (int64_t)threadIdx.x * kVec;
#pragma unroll
  for (int j = 0; j < kUnroll; ++j) {
    const int64_t e = base + (int64_t)j * kSlab;
    if (e >= n) continue;
    const anc_f32x4 p = anc_ld_stream((const anc_f32x4 *)(p32 + e));
    const float pp[4] = {p.x, p.y, p.z, p.w};
    uint32_t hb[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const uint64_t i = (uint64_t)(e + k);
      hb[k] = SR ? anc_bf16_sr_bits(pp[k], (uint32_t)(i >> 6), (uint32_t)(i & 63u), seed)
                 : anc_bf16_rne_bits(pp[k]);
    }
    anc_u32x2 ho = {(hb[0] & 0xFFFFu) | (hb[1] << 16), (hb[2] & 0xFFFFu) | (hb[3] << 16)};
    anc_st_stream((anc_u32x2 *)(p16 + e), ho);
  }
}


// ---- row-sparse AdamW, dense-equivalent ---------------------------------------------------
// For a (V, H) tensor whose gradient touches few rows per step (an input embedding that is not
// tied to the output head). A dense step on a row with zero gradient still moves it (m and v decay,
// the bias-corrected momentum and the weight decay keep updating p), so skipping untouched rows
// changes the result; instead every row remembers the last step it is current for, and when it is
// next needed the steps it missed are replayed on it, each with g = 0 and that step's own scalars
// (bias corrections, learning rate, rounding seed) from a per-step table, through the same
// per-element routine as the dense kernel. The state of a row that is current is therefore
// bit-identical to what the dense kernel would hold. A row is brought up to date (a) before the
// forward pass gathers it (anc_adamw_rows with grads = 0: replay through step t_now) and (b) by
// the step itself (replay through t_now - 1, then step t_now with its gradient row).
template <int FORM, int SR>
__global__ void __launch_bounds__(kThreads)
k_adamw_rows(const int32_t *__restrict__ rows, const float *__restrict__ grads, float *__restrict__ m,
             float *__restrict__ v, float *__restrict__ p32, uint16_t *__restrict__ p16,
             int32_t *__restrict__ last, int H, int64_t V, const RowStep *__restrict__ table, int t_now,
             anc_adamw_hyper_t h, float wd, uint32_t seed, const anc_step_ctl_t *__restrict__ ctl) {
  float clip;
  if (!load_ctl(ctl, clip)) return;                      // skipped step: nothing is touched
  const int64_t row = rows != nullptr ? (int64_t)rows[blockIdx.x] : (int64_t)blockIdx.x;
  if (row < 0 || row >= V) return;
  const int k0 = last[row];
  __syncthreads();                                       // every lane has read `last` before lane 0 rewrites it
  const bool with_step = grads != nullptr;
  const int t_replay = with_step ? t_now - 1 : t_now;    // replay (g = 0) through this step
  if (k0 >= t_now || (!with_step && k0 >= t_replay)) return;
  for (int c = (int)threadIdx.x * kVec; c < H; c += kSlab) {
    const int64_t e = row * H + c;
    const anc_f32x4 m4 = *(const anc_f32x4 *)(m + e), v4 = *(const anc_f32x4 *)(v + e), p4 = *(const anc_f32x4 *)(p32 + e);
    float mm[4] = {m4.x, m4.y, m4.z, m4.w}, vv[4] = {v4.x, v4.y, v4.z, v4.w}, pp[4] = {p4.x, p4.y, p4.z, p4.w};
    anc_adamw_hyper_t hs = h;
    uint32_t seed_step = 0;
    for (int s = k0 + 1; s <= t_replay; ++s) {
      const RowStep rs = table[s];
      hs.bc1 = rs.bc1; hs.bc2 = rs.bc2; hs.lr = rs.lr;
      seed_step = rs.seed_base;
#pragma unroll
      for (int k = 0; k < 4; ++k) adamw_elem<FORM>(0.0f, mm[k], vv[k], pp[k], hs, wd, 1.0f);
    }
    if (with_step) {
      const RowStep rs = table[t_now];
      hs.bc1 = rs.bc1; hs.bc2 = rs.bc2; hs.lr = rs.lr;
      seed_step = rs.seed_base;
      const anc_f32x4 g4 = *(const anc_f32x4 *)(grads + (int64_t)blockIdx.x * H + c);
      const float gg[4] = {g4.x, g4.y, g4.z, g4.w};
#pragma unroll
      for (int k = 0; k < 4; ++k) adamw_elem<FORM>(gg[k], mm[k], vv[k], pp[k], hs, wd, clip);
    }
    uint32_t hb[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const uint64_t i = (uint64_t)(e + k);
      hb[k] = SR ? anc_bf16_sr_bits(pp[k], (uint32_t)(i >> 6), (uint32_t)(i & 63u), seed_step + seed)
                 : anc_bf16_rne_bits(pp[k]);
    }
    *(anc_f32x4 *)(m + e) = anc_f32x4{mm[0], mm[1], mm[2], mm[3]};
    *(anc_f32x4 *)(v + e) = anc_f32x4{vv[0], vv[1], vv[2], vv[3]};
    *(anc_f32x4 *)(p32 + e) = anc_f32x4{pp[0], pp[1], pp[2], pp[3]};
    *(anc_u32x2 *)(p16 + e) = anc_u32x2{(hb[0] & 0xFFFFu) | (hb[1] << 16), (hb[2] & 0xFFFFu) | (hb[3] << 16)};
  }
  if (threadIdx.x == 0) last[row] = t_now;
}

int check_hyper(const anc_adamw_hyper_t *h, const char *who) {
  ANC_REQUIRE(h != nullptr, "%s: null hyper-parameter block", who);
  ANC_REQUIRE(h->form == ANC_ADAMW_FORM_DIV || h->form == ANC_ADAMW_FORM_IBC,
              "%s: unknown form %d", who, h->form);
  ANC_REQUIRE(h->sr == 0 || h->sr == ANC_SR_ON || h->sr == (ANC_SR_ON | ANC_SR_STEP_SEED),
              "%s: sr must be 0, ANC_SR_ON or ANC_SR_ON | ANC_SR_STEP_SEED", who);
  ANC_REQUIRE(h->step_table == 0 || ((h->step_table & 15) == 0 && h->step_cap >= 1),
              "%s: step_table must be 16-byte aligned with step_cap >= 1", who);
  return ANC_OK;
}

}  // namespace

extern "C" int64_t anc_adamw_num_blocks(int64_t n) {
  return n <= 0 ? 0 : (n + kBlockElems - 1) / kBlockElems;
}

// Turn the runtime (form, sr) pair into template arguments.
template <int V> struct IC { static constexpr int value = V; };
template <typename F> static void dispatch_form_sr(int form, int sr, F &&f) {
  if (form == ANC_ADAMW_FORM_DIV) {
    if (sr) f(IC<ANC_ADAMW_FORM_DIV>{}, IC<1>{}); else f(IC<ANC_ADAMW_FORM_DIV>{}, IC<0>{});
  } else {
    if (sr) f(IC<ANC_ADAMW_FORM_IBC>{}, IC<1>{}); else f(IC<ANC_ADAMW_FORM_IBC>{}, IC<0>{});
  }
}

extern "C" int anc_adamw(uint64_t g, uint64_t m, uint64_t v, uint64_t p32, uint64_t p16,
                         int64_t n, int g_dtype, const anc_adamw_hyper_t *h, float wd,
                         uint32_t seed, uint64_t ctl, uint64_t stream) {
  if (int rc = check_hyper(h, "anc_adamw")) return rc;
  ANC_REQUIRE(ctl != 0 || (h->step_table == 0 && !(h->sr & ANC_SR_STEP_SEED)),
              "anc_adamw: steps counted on the device need the control block");
  ANC_REQUIRE(g && m && v && p32 && p16, "anc_adamw: null device pointer");
  ANC_REQUIRE(n > 0 && n % 64 == 0, "anc_adamw: n=%lld must be a positive multiple of 64",
              (long long)n);
  ANC_REQUIRE(g_dtype == ANC_F32 || g_dtype == ANC_BF16, "anc_adamw: bad g_dtype %d", g_dtype);
  ANC_REQUIRE(((m | v | p32) & 15) == 0 && (p16 & 7) == 0 &&
                  (g & (g_dtype == ANC_F32 ? 15 : 7)) == 0,
              "anc_adamw: pointers must be 16-byte aligned (8 for bf16 tensors)");
  const int64_t blocks = anc_adamw_num_blocks(n);
  ANC_REQUIRE(blocks < (1ll << 31), "anc_adamw: tensor too large for one launch");
  Tensor t{(const void *)g, (float *)m, (float *)v, (float *)p32, (uint16_t *)p16, n, wd,
           h->seed_base + seed};
  const anc_step_ctl_t *c = (const anc_step_ctl_t *)ctl;
  const anc_adamw_hyper_t hh = *h;
  AncProfScope prof(ANC_PROF_ADAMW, anc_stream(stream));
  dispatch_form_sr(hh.form, hh.sr, [&](auto F, auto S) {
    constexpr int f = decltype(F)::value, s = decltype(S)::value;
    if (g_dtype == ANC_BF16)
      hipLaunchKernelGGL((k_adamw<ANC_BF16, f, s>), dim3((unsigned)blocks), dim3(kThreads), 0,
                         anc_stream(stream), t, hh, c);
    else
      hipLaunchKernelGGL((k_adamw<ANC_F32, f, s>), dim3((unsigned)blocks), dim3(kThreads), 0,
                         anc_stream(stream), t, hh, c);
  });
  ANC_LAUNCH_CHECK();
  return ANC_OK;
}

extern "C" int anc_adamw_multi(uint64_t desc_table, int32_t n_tensors, int64_t total_blocks,
                               const anc_adamw_hyper_t *h, uint64_t ctl, uint64_t stream) {
  if (int rc = check_hyper(h, "anc_adamw_multi")) return rc;
  ANC_REQUIRE(ctl != 0 || (h->step_table == 0 && !(h->sr & ANC_SR_STEP_SEED)),
              "anc_adamw_multi: steps counted on the device need the control block");
  ANC_REQUIRE(desc_table != 0 && n_tensors > 0, "anc_adamw_multi: empty descriptor table");
  ANC_REQUIRE(total_blocks > 0 && total_blocks < (1ll << 31),
              "anc_adamw_multi: total_blocks=%lld out of range", (long long)total_blocks);
  const anc_adamw_desc_t *tab = (const anc_adamw_desc_t *)desc_table;
  const anc_step_ctl_t *c = (const anc_step_ctl_t *)ctl;
  const anc_adamw_hyper_t hh = *h;
  AncProfScope prof(ANC_PROF_ADAMW, anc_stream(stream));
  dispatch_form_sr(hh.form, hh.sr, [&](auto F, auto S) {
    constexpr int f = decltype(F)::value, s = decltype(S)::value;
    hipLaunchKernelGGL((k_adamw_multi<f, s>), dim3((unsigned)total_blocks), dim3(kThreads), 0,
                       anc_stream(stream), tab, (int)n_tensors, hh, c);
  });
  ANC_LAUNCH_CHECK();
  return ANC_OK;
}

// Row-sparse AdamW on a (V, H) tensor (see k_adamw_rows). rows: n_rows distinct row indices
// (int32, device) or 0 for "every row, in order" (n_rows = V). grads: (n_rows, H) fp32, row i the
// gradient of rows[i], or 0 to bring the rows up to date through step t_now without a step.
// step_table: device array of {bc1, bc2, lr, seed_base} per counted step, entries 1 .. t_now.
extern "C" int anc_adamw_rows(uint64_t rows, int64_t n_rows, uint64_t grads, uint64_t m, uint64_t v,
                              uint64_t p32, uint64_t p16, uint64_t last_step, int64_t V, int64_t H,
                              uint64_t step_table, int32_t t_now, const anc_adamw_hyper_t *h, float wd,
                              uint32_t seed, uint64_t ctl, uint64_t stream) {
  if (int rc = check_hyper(h, "anc_adamw_rows")) return rc;
  ANC_REQUIRE(m && v && p32 && p16 && last_step && step_table, "anc_adamw_rows: null device pointer");
  ANC_REQUIRE(V > 0 && H > 0 && H % 64 == 0 && n_rows > 0 && n_rows < (1ll << 31) && (rows != 0 || n_rows == V),
              "anc_adamw_rows: V=%lld, H=%lld (multiple of 64), n_rows=%lld", (long long)V, (long long)H,
              (long long)n_rows);
  ANC_REQUIRE(t_now >= 1, "anc_adamw_rows: t_now=%d: steps count from 1", t_now);
  ANC_REQUIRE(((m | v | p32 | grads | step_table) & 15) == 0 && (p16 & 7) == 0 && ((rows | last_step) & 3) == 0,
              "anc_adamw_rows: misaligned pointers");
  const anc_adamw_hyper_t hh = *h;
  AncProfScope prof(ANC_PROF_ADAMW, anc_stream(stream));
  dispatch_form_sr(hh.form, hh.sr, [&](auto F, auto S) {
    constexpr int f = decltype(F)::value, s = decltype(S)::value;
    hipLaunchKernelGGL((k_adamw_rows<f, s>), dim3((unsigned)n_rows), dim3(kThreads), 0, anc_stream(stream),
                       (const int32_t *)rows, (const float *)grads, (float *)m, (float *)v, (float *)p32,
                       (uint16_t *)p16, (int32_t *)last_step, (int)H, V, (const RowStep *)step_table, (int)t_now, hh,
                       wd, seed, (const anc_step_ctl_t *)ctl);
  });
  ANC_LAUNCH_CHECK();
  return ANC_OK;
}

extern "C" int anc_cast_bf16(uint64_t p32, uint64_t p16, int64_t n, int sr, uint32_t seed,
                             uint64_t stream) {
  ANC_REQUIRE(p32 && p16 && n > 0 && n % 4 == 0, "anc_cast_bf16: bad arguments (n=%lld)",
              (long long)n);
  ANC_REQUIRE((p32 & 15) == 0 && (p16 & 7) == 0, "anc_cast_bf16: misaligned pointers");
  const int64_t blocks = (n + kBlockElems - 1) / kBlockElems;
  ANC_REQUIRE(blocks < (1ll << 31), "anc_cast_bf16: tensor too large for one launch");
  AncProfScope prof(ANC_PROF_MISC, anc_stream(stream));
  if (sr)
    hipLaunchKernelGGL(k_cast_bf16<1>, dim3((unsigned)blocks), dim3(kThreads), 0, anc_stream(stream),
                       (const float *)p32, (uint16_t *)p16, n, seed);
  else
    hipLaunchKernelGGL(k_cast_bf16<0>, dim3((unsigned)blocks), dim3(kThreads), 0, anc_stream(stream),
                       (const float *)p32, (uint16_t *)p16, n, seed);
  ANC_LAUNCH_CHECK();
  return ANC_OK;
}
