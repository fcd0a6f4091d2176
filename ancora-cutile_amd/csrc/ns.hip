// Batched Newton-Schulz / Polar-Express chain for gfx950.
// Replaces `newton_schulz_resident[_e]` and the kernels they launch
// (ancora/kernels/muon_ns.py:68-174, 245-283, 293-406, 430-468); numpy form
// ancora/optim/muon.py:67-80 and tests/kernels/_probe_polar_express_device.py:27-34.
//
// Per matrix X (M,N), M <= N:  X /= ||X||_F + eps;  steps x { A = X X^T;
//   B = b A + c A A;  X = a X + B X }.
//
// Precision design (bf16 modes). The reference stores X, A and B as bf16 between the
// GEMMs, which leaves it about 6e-3 (relative Frobenius) from the fp32 numpy result.
// Here the iterate is carried between steps as a bf16 pair X = Xh + Xl (Xh = bf16(x),
// Xl = bf16(x - Xh): 16 significant bits, 4 bytes per element like fp32 but directly usable
// as matrix-core operands), and the diagonals of A and B -- the entries that approach 1 and
// b+c while the off-diagonal part goes to zero -- never pass through bf16:
//   A = dA + F    dA = diag(A) kept as an fp32 vector, F = off-diagonal part
//   A A = dA^2 + dA F + F dA + F F       only F F is a matrix-core product (bf16 F)
//   B = dB + Boff                        likewise
//   B X = dB (.) X + Boff X              dB (.) X is an fp32 row scaling in the epilogue
// Xh alone is the matrix-core operand of the early iterations. Where the shape needs it (see
// split_plan below) late iterations add the residual products: A gets Xh Xl^T + Xl Xh^T and
// B X gets Boff Xl as extra accumulation terms of the same tile. The symmetric products are
// "NT" (both operands K-contiguous rows of X or F); B X reads the iterate as (k, n) tiles
// and transposes inside LDS reads, so no transposed copy of X exists. The 256-tile kernels
// keep every matrix the chain writes for itself in panel layout (32-column panels, see NsGemm);
// the input pair and everything the 128-tile kernels touch is row-major. The
// fp32 input is read once (normalisation) and the fp32 result written once (last step).
//
// Determinism: one workgroup owns one 128x128 output tile and its whole K loop, terms in
// a fixed order, K tiles in ascending order; no split-K, no atomics. A matrix's result
// does not depend on the batch size E or on its position in the batch. Symmetric outputs
// (A, B) compute the tiles on or below the diagonal and mirror them; without residual terms
// that is bit-identical to computing both halves (same products, same order, and an epilogue
// that is symmetric in (i,j)). With residual terms the two cross products Xh Xl^T and
// Xl Xh^T enter one accumulator in a fixed order, so elements computed directly inside a
// diagonal tile differ from their mirror images in the last bits; nothing depends on it.
//
// GEMM tile: 128x128x64, 256 lanes = 4 wavefronts in 2x2, each 64x64 as 2x2
// v_mfma_f32_32x32x16_bf16 blocks (fp32 accumulate). Operand tiles are staged through LDS
// with a 144-byte row pitch (16-byte fragment reads of 16 consecutive rows hit 64 distinct
// banks); the next K tile is fetched into registers while the current one is multiplied.
// Workgroup ids are remapped so that consecutive tiles -- the tiles of one matrix -- run on
// the same XCD and share its L2.
#include <vector>

#include "reduce.h"
#include "ns_common.h"

namespace {

using namespace anc_reduce;

// bf16 (round to nearest even) by the hardware conversion, as in the 256-tile kernel
__device__ __forceinline__ uint32_t hw_bf16(float x) { return anc_pk_bf16(x, 0.0f) & 0xFFFFu; }

template <int EPI>
__global__ void __launch_bounds__(kGemmThreads, 2) k_ns_gemm(NsGemm p) {
  __shared__ __attribute__((aligned(16))) uint16_t sA[BM * PITCH];
  // B tile: [n][k] rows of PITCH for the symmetric products; [k][n] rows of NPITCH (320 bytes:
  // consecutive rows start 64 bytes apart in the banks) for X = a X + B X, which reads the
  // iterate (K, N) row-major as it lies in memory and transposes while reading fragments.
  constexpr int NPITCH = BN + 32;
  constexpr bool BT = (EPI == EPI_BX);
  __shared__ __attribute__((aligned(16))) uint16_t sB[BT ? BK * NPITCH : BN * PITCH];

  const int L = xcd_remap((int)blockIdx.x, (int)gridDim.x);
  const int tiles_per = p.lower ? p.tiles_m * (p.tiles_m + 1) / 2 : p.tiles_m * p.tiles_n;
  const int e = L / tiles_per;
  const int t = L % tiles_per;
  int tm, tn;
  if (p.lower) {
    tm = 0;
    while ((tm + 1) * (tm + 2) / 2 <= t) ++tm;
    tn = t - tm * (tm + 1) / 2;
  } else {
    tm = t / p.tiles_n;
    tn = t % p.tiles_n;
  }

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int lrow = tid >> 3, lk = (tid & 7) * 8;     // loader: 8 lanes per 128-byte row
  const int K = p.K;
  const int nk = K / BK;
  const int total = anc_ns_terms(p, e) * nk;

  f32x16 acc[2][2];
#pragma unroll
  for (int bi = 0; bi < 2; ++bi)
#pragma unroll
    for (int bj = 0; bj < 2; ++bj)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[bi][bj][r] = 0.0f;

  anc_u32x4 ra[4], rb[4];
  auto gload = [&](int step) {
    const int term = step / nk, kt = step - term * nk;
    const uint16_t *Ap = p.A[term] + (int64_t)e * p.strideA + (int64_t)(tm * BM + lrow) * K + kt * BK + lk;
    // (k, n) tile: 16 lanes per 256-byte row, 16 rows per pass
    const uint16_t *Bp = BT ? p.B[term] + (int64_t)e * p.strideB + (int64_t)(kt * BK + (tid >> 4)) * p.N + tn * BN + (tid & 15) * 8
                            : p.B[term] + (int64_t)e * p.strideB + (int64_t)(tn * BN + lrow) * K + kt * BK + lk;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      ra[i] = *(const anc_u32x4 *)(Ap + (int64_t)(32 * i) * K);
      rb[i] = BT ? *(const anc_u32x4 *)(Bp + (int64_t)(16 * i) * p.N) : *(const anc_u32x4 *)(Bp + (int64_t)(32 * i) * K);
    }
  };
  auto lstore = [&]() {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      *(anc_u32x4 *)&sA[(lrow + 32 * i) * PITCH + lk] = ra[i];
      if (BT) *(anc_u32x4 *)&sB[((tid >> 4) + 16 * i) * NPITCH + (tid & 15) * 8] = rb[i];
      else *(anc_u32x4 *)&sB[(lrow + 32 * i) * PITCH + lk] = rb[i];
    }
  };

  gload(0);
  lstore();
  __syncthreads();
  const int arow = (wm * 64 + (lane & 31)) * PITCH + (lane >> 5) * 8;
  const int brow = (wn * 64 + (lane & 31)) * PITCH + (lane >> 5) * 8;
  // transposing reads: lane s of each 16-lane group addresses row s/4, columns 4*(s%4)..+3
  const int btr = (8 * (lane >> 5) + ((lane & 15) >> 2)) * NPITCH + wn * 64 + 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
  for (int step = 0; step < total; ++step) {
    const bool more = step + 1 < total;
    if (more) gload(step + 1);
#pragma unroll
    for (int kk = 0; kk < BK / 16; ++kk) {
      bf16x8 a[2], b[2];
#pragma unroll
      for (int bi = 0; bi < 2; ++bi) a[bi] = *(const bf16x8 *)&sA[arow + bi * 32 * PITCH + kk * 16];
#pragma unroll
      for (int bj = 0; bj < 2; ++bj)
        b[bj] = BT ? anc_lds_tr_frag(&sB[btr + kk * 16 * NPITCH + bj * 32], &sB[btr + (kk * 16 + 4) * NPITCH + bj * 32])
                   : *(const bf16x8 *)&sB[brow + bj * 32 * PITCH + kk * 16];
#pragma unroll
      for (int bi = 0; bi < 2; ++bi)
#pragma unroll
        for (int bj = 0; bj < 2; ++bj)
          acc[bi][bj] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[bi], b[bj], acc[bi][bj], 0, 0, 0);
    }
    __syncthreads();
    if (more) {
      lstore();
      __syncthreads();
    }
  }

  // ---- epilogue. Accumulator element r of block (bi,bj) in lane l is
  //      row 8*(r/4) + 4*(l/32) + r%4, column l%32 of the 32x32 block.
  const int M = p.M, N = p.N;
  const int64_t mm = (int64_t)e * M * M, mn = (int64_t)e * M * N, mv = (int64_t)e * M;
  float sc = 1.0f;
  if (EPI != EPI_BMAT && p.scale != nullptr) sc = p.scale[e];
  const float acc_scale = (EPI == EPI_GRAM) ? sc * sc : sc;
  const bool has_a32 = EPI != EPI_BX && anc_ns_has_a32(p, e);
#pragma unroll
  for (int bi = 0; bi < 2; ++bi) {
#pragma unroll
    for (int bj = 0; bj < 2; ++bj) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int gi = tm * BM + wm * 64 + bi * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
        const int gj = tn * BN + wn * 64 + bj * 32 + (lane & 31);
        const float v = (EPI == EPI_BMAT) ? acc[bi][bj][r] : acc[bi][bj][r] * acc_scale;
        if (EPI == EPI_GRAM) {
          const bool diag = gi == gj;
          const uint16_t fh = diag ? (uint16_t)0 : (uint16_t)hw_bf16(v);
          if (has_a32) p.A32[mm + (int64_t)gi * M + gj] = v;
          p.Fh[mm + (int64_t)gi * M + gj] = fh;
          if (tm != tn) {
            if (has_a32) p.A32[mm + (int64_t)gj * M + gi] = v;
            p.Fh[mm + (int64_t)gj * M + gi] = fh;
          }
          if (p.Fl != nullptr) {
            const uint16_t fl =
                diag ? (uint16_t)0 : (uint16_t)hw_bf16(v - anc_bf16_bits_to_f32(fh));
            p.Fl[mm + (int64_t)gi * M + gj] = fl;
            if (tm != tn) p.Fl[mm + (int64_t)gj * M + gi] = fl;
          }
          if (diag) p.dA[mv + gi] = v;
        } else if (EPI == EPI_BMAT) {
          const float a = has_a32 ? p.A32[mm + (int64_t)gi * M + gj]
                                  : anc_bf16_bits_to_f32(p.Fh[mm + (int64_t)gi * M + gj]);
          const float di = p.dA[mv + gi], dj = p.dA[mv + gj];
          uint16_t bh, bl = 0;
          if (gi != gj) {
            const float a2 = v + (di * a + a * dj);   // symmetric in (i,j)
            const float bv = p.cb * a + p.cc * a2;
            bh = (uint16_t)hw_bf16(bv);
            bl = (uint16_t)hw_bf16(bv - anc_bf16_bits_to_f32(bh));
          } else {
            const float a2 = v + di * di;
            p.dB[mv + gi] = p.cb * di + p.cc * a2;
            bh = 0;
          }
          p.Bh[mm + (int64_t)gi * M + gj] = bh;
          if (tm != tn) p.Bh[mm + (int64_t)gj * M + gi] = bh;
          if (p.Bl != nullptr) {
            p.Bl[mm + (int64_t)gi * M + gj] = bl;
            if (tm != tn) p.Bl[mm + (int64_t)gj * M + gi] = bl;
          }
        } else {
          const int64_t o = mn + (int64_t)gi * N + gj;
          const float x = (anc_bf16_bits_to_f32(p.Xh[o]) + anc_bf16_bits_to_f32(p.Xl[o])) * sc;
          const float y = (p.ca + p.dB[mv + gi]) * x + v;
          if (p.X32 != nullptr) p.X32[o] = y;
          if (p.Yh != nullptr) {
            const uint32_t yh = hw_bf16(y);
            p.Yh[o] = (uint16_t)yh;
            p.Yl[o] = (uint16_t)hw_bf16(y - anc_bf16_bits_to_f32(yh));
          }
        }
      }
    }
  }
}

// ---------------------------------------------------------------- fp32 validation GEMM
// 128x128x16 tiles, v_mfma_f32_32x32x2_f32: every product and every sum in fp32.
constexpr int FK = 16, FPITCH = 20, FNPITCH = 132;

struct NsGemmF32 {
  const float *A;          // (E, Mo, K) rows of the output
  const float *B;          // NT: (E, No, K);  NN: (E, K, No)
  int K, nn;
  int64_t strideA, strideB;
  int Mo, No;              // output dims per matrix
  float ca, cb, cc;
  const float *D;          // epilogue operand, same shape as the output (may be null)
  float *out;
  int epi;
};

__global__ void __launch_bounds__(kGemmThreads, 2) k_ns_gemm_f32(NsGemmF32 p) {
  __shared__ __attribute__((aligned(16))) float sA[BM * FPITCH];
  __shared__ __attribute__((aligned(16))) float sB[BM * FPITCH > FK * FNPITCH ? BM * FPITCH : FK * FNPITCH];
  const int tiles_m = p.Mo / BM, tiles_n = p.No / BN;
  const int L = xcd_remap((int)blockIdx.x, (int)gridDim.x);
  const int e = L / (tiles_m * tiles_n), t = L % (tiles_m * tiles_n);
  const int tm = t / tiles_n, tn = t % tiles_n;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int K = p.K;

  f32x16 acc[2][2];
#pragma unroll
  for (int bi = 0; bi < 2; ++bi)
#pragma unroll
    for (int bj = 0; bj < 2; ++bj)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[bi][bj][r] = 0.0f;

  const float *Ae = p.A + (int64_t)e * p.strideA + (int64_t)(tm * BM) * K;
  const float *Be = p.B + (int64_t)e * p.strideB;
  for (int k0 = 0; k0 < K; k0 += FK) {
    // A tile: 128 rows x 16 k, 4 lanes per row
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int row = (tid >> 2) + 64 * i, kq = (tid & 3) * 4;
      *(anc_f32x4 *)&sA[row * FPITCH + kq] = *(const anc_f32x4 *)(Ae + (int64_t)row * K + k0 + kq);
    }
    if (!p.nn) {
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const int row = (tid >> 2) + 64 * i, kq = (tid & 3) * 4;
        *(anc_f32x4 *)&sB[row * FPITCH + kq] =
            *(const anc_f32x4 *)(Be + (int64_t)(tn * BN + row) * K + k0 + kq);
      }
    } else {
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const int kr = (tid >> 5) + 8 * i, c4 = (tid & 31) * 4;
        *(anc_f32x4 *)&sB[kr * FNPITCH + c4] =
            *(const anc_f32x4 *)(Be + (int64_t)(k0 + kr) * p.No + tn * BN + c4);
      }
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < FK / 2; ++kk) {
      float a[2], b[2];
      const int kx = kk * 2 + (lane >> 5);
#pragma unroll
      for (int bi = 0; bi < 2; ++bi) a[bi] = sA[(wm * 64 + bi * 32 + (lane & 31)) * FPITCH + kx];
#pragma unroll
      for (int bj = 0; bj < 2; ++bj)
        b[bj] = p.nn ? sB[kx * FNPITCH + wn * 64 + bj * 32 + (lane & 31)]
                     : sB[(wn * 64 + bj * 32 + (lane & 31)) * FPITCH + kx];
#pragma unroll
      for (int bi = 0; bi < 2; ++bi)
#pragma unroll
        for (int bj = 0; bj < 2; ++bj)
          acc[bi][bj] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[bi], b[bj], acc[bi][bj], 0, 0, 0);
    }
    __syncthreads();
  }
  const int64_t base = (int64_t)e * p.Mo * p.No;
#pragma unroll
  for (int bi = 0; bi < 2; ++bi)
#pragma unroll
    for (int bj = 0; bj < 2; ++bj)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int gi = tm * BM + wm * 64 + bi * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
        const int gj = tn * BN + wn * 64 + bj * 32 + (lane & 31);
        const int64_t o = base + (int64_t)gi * p.No + gj;
        const float v = acc[bi][bj][r];
        float y;
        if (p.epi == EPI_GRAM)      y = v;
        else if (p.epi == EPI_BMAT) y = p.cb * p.D[o] + p.cc * v;
        else                        y = p.ca * p.D[o] + v;
        p.out[o] = y;
      }
}

// ------------------------------------------------------------------ Frobenius prologue
__global__ void __launch_bounds__(kThreads)
k_fro_partials(const float *__restrict__ X, int64_t mn, int nchunks, double *__restrict__ partials) {
  const int64_t e = (int64_t)blockIdx.x / nchunks, c = (int64_t)blockIdx.x % nchunks;
  chunk_partial<ANC_F32>((const void *)(X + e * mn), mn, c, partials + blockIdx.x);
}

// One block per matrix: lane t adds partials t, t+256, ... in order; butterfly; 4 wavefronts in order.
// pow2 (pair entries only, else null): a matrix whose sum of squares is below 2^-100 (products of
// its elements would underflow fp32 in the first A = U U^T) gets pow2[e] = 2^k with 2^k ||U|| in
// [1, 2), every other matrix 1; k_pair_rescale multiplies the pair by it (exact) and the
// reciprocal carries 2^-k, so the first step sees the same scale*U as without.
__global__ void __launch_bounds__(kThreads)
k_fro_finalize(const double *__restrict__ partials, int nchunks, float eps, float *__restrict__ recip,
               float *__restrict__ pow2) {
  __shared__ double wave_sum[kThreads / 64];
  const double *p = partials + (int64_t)blockIdx.x * nchunks;
  double acc = 0.0;
  for (int i = threadIdx.x; i < nchunks; i += kThreads) acc = acc + p[i];
  acc = anc_wave_sum_f64(acc);
  if ((threadIdx.x & 63) == 0) wave_sum[threadIdx.x >> 6] = acc;
  __syncthreads();
  if (threadIdx.x == 0) {
    double t = wave_sum[0];
#pragma unroll
    for (int w = 1; w < kThreads / 64; ++w) t = t + wave_sum[w];
    float r = 1.0f / ((float)sqrt(t) + eps);
    if (pow2 != nullptr) {
      float sc = 1.0f;
      if (t > 0.0 && t < 0x1p-100) {
        const int k = -ilogb(sqrt(t));
        sc = ldexpf(1.0f, k);
        r = ldexpf(r, -k);
      }
      pow2[blockIdx.x] = sc;
    }
    recip[blockIdx.x] = r;
  }
}

// Multiply the bf16 pair of every matrix whose pow2 is not 1 by it (exact). One workgroup per
// matrix: it returns at once unless its matrix is one of the rare tiny ones.
__global__ void __launch_bounds__(kThreads)
k_pair_rescale(uint16_t *__restrict__ Uh, uint16_t *__restrict__ Ul, const float *__restrict__ pow2, int64_t mn) {
  const float sc = pow2[blockIdx.x];
  if (sc == 1.0f) return;
  for (int64_t o = (int64_t)threadIdx.x * 8; o < mn; o += (int64_t)kThreads * 8) {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      uint16_t *p = (h ? Ul : Uh) + (int64_t)blockIdx.x * mn + o;
      anc_u32x4 w = *(const anc_u32x4 *)p;
      uint32_t q[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float lo = __uint_as_float(q[i] << 16) * sc, hi = __uint_as_float(q[i] & 0xFFFF0000u) * sc;
        q[i] = (__float_as_uint(lo) >> 16) | (__float_as_uint(hi) & 0xFFFF0000u);
      }
      *(anc_u32x4 *)p = anc_u32x4{q[0], q[1], q[2], q[3]};
    }
  }
}

// Normalisation X * recip[e]. With Xh == null the fp32 matrix is scaled in place (fp32 chain,
// steps == 0); otherwise X is left alone and the scaled iterate leaves as the bf16 pair
// Xh = bf16(x), Xl = bf16(x - Xh), both (M,N) row-major. 8 elements per lane.
__global__ void __launch_bounds__(kThreads)
k_ns_prep(float *__restrict__ X, const float *__restrict__ recip, int64_t mn, int64_t total8,
          uint16_t *__restrict__ Xh, uint16_t *__restrict__ Xl) {
  const int64_t i8 = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  if (i8 >= total8) return;
  const int64_t o = i8 * 8;
  const float rc = recip[o / mn];
  const anc_f32x4 x0 = anc_ld_stream((const anc_f32x4 *)(X + o));
  const anc_f32x4 x1 = anc_ld_stream((const anc_f32x4 *)(X + o + 4));
  const float xs[8] = {x0.x * rc, x0.y * rc, x0.z * rc, x0.w * rc, x1.x * rc, x1.y * rc, x1.z * rc, x1.w * rc};
  if (Xh == nullptr) {
    const anc_f32x4 y0 = {xs[0], xs[1], xs[2], xs[3]}, y1 = {xs[4], xs[5], xs[6], xs[7]};
    *(anc_f32x4 *)(X + o) = y0;
    *(anc_f32x4 *)(X + o + 4) = y1;
    return;
  }
  uint32_t h[8], l[8];
#pragma unroll
  for (int k = 0; k < 8; ++k) {
    h[k] = anc_bf16_rne_bits(xs[k]) & 0xFFFFu;
    l[k] = anc_bf16_rne_bits(xs[k] - anc_bf16_bits_to_f32(h[k])) & 0xFFFFu;
  }
  const anc_u32x4 ho = {h[0] | (h[1] << 16), h[2] | (h[3] << 16), h[4] | (h[5] << 16), h[6] | (h[7] << 16)};
  const anc_u32x4 lo = {l[0] | (l[1] << 16), l[2] | (l[3] << 16), l[4] | (l[5] << 16), l[6] | (l[7] << 16)};
  anc_st_stream((anc_u32x4 *)(Xh + o), ho);
  anc_st_stream((anc_u32x4 *)(Xl + o), lo);
}

// ------------------------------------------------------------------ conditioning proxy
// ||offdiag(A)||_F^2 of the first iteration's A = X X^T (||X||_F = 1, so tr A = 1): 1/N for a
// matrix with independent entries whatever its row scaling, N/r - N/M for one whose mass sits
// in r directions that are spread over the rows (outlier columns). Read from Fh (bf16, zero
// diagonal). kCondParts blocks per matrix, each over M*M/kCondParts consecutive elements: lane t
// takes the 8-element vectors t, t+256, ..., adds their squares left to right in fp32, widens to
// fp64; butterfly over the wavefront; the 4 wavefront sums in order. The consumers add the
// kCondParts partial sums in order (anc_ns_terms).
struct NsCondArgs {
  int n;
  int blocks[kMaxGroups];
  const uint16_t *Fh[kMaxGroups];
  double *out[kMaxGroups];
  int M[kMaxGroups];
};
__global__ void __launch_bounds__(kThreads) k_ns_cond(NsCondArgs a) {
  __shared__ double wave_sum[kThreads / 64];
  int b = (int)blockIdx.x, q = 0;
  while (q + 1 < a.n && b >= a.blocks[q]) { b -= a.blocks[q]; ++q; }
  const int64_t per = (int64_t)a.M[q] * a.M[q] / kCondParts;
  const uint16_t *src = a.Fh[q] + (int64_t)b * per;          // b = e * kCondParts + part
  double acc = 0.0;
  for (int64_t v = threadIdx.x; v < per / kRun; v += kThreads) acc = acc + (double)run_sumsq<ANC_BF16>(src, v * kRun, per);
  acc = anc_wave_sum_f64(acc);
  if ((threadIdx.x & 63) == 0) wave_sum[threadIdx.x >> 6] = acc;
  __syncthreads();
  if (threadIdx.x == 0) {
    double t = wave_sum[0];
#pragma unroll
    for (int w = 1; w < kThreads / 64; ++w) t = t + wave_sum[w];
    a.out[q][b] = t;
  }
}

// ------------------------------------------------------------------ column statistic, classification
// The proxy cannot tell a few huge COLUMNS (N/r of them: 1 % of the columns x100 reads 100 whatever
// N) from a low-rank signal over weak noise (rank 32: N/32), and the two need different plans: the
// first meets the bar with the cheap gates, the second only with every residual term (rank 32 plus
// 10 % noise at 1024x2048: 2.9e-3 against 1.4e-4). What separates them is where the mass sits among
// the columns: colc = N * sum_j c_j^4 / (sum_j c_j^2)^2 over the column norms c_j of the input
// (taken over every fourth row) is N/r for r outlier columns (equal to the proxy) and 1.0 .. 1.5
// for anything rotationally spread.
// The same statistic separates, just below the band, scaled columns (colc = proxy: the low gate
// suffices) from a spectrum with a gap (colc = 1: near-duplicate rows, 2.4e-3 at 1024x1024 without
// the wide gate's terms, 4.6e-4 with).
// k_ns_colstat: one block per 64 columns of a matrix; 8 lanes cover a 128-byte row piece with
// 16-byte loads, the 32 row groups walk the M rows (fp64 sums of squares: the pair entries run on
// unnormalised input) and are added in order through LDS; the block leaves (sum c^2, sum c^4) of
// its columns (one wavefront's butterfly). A block returns at
// once unless the matrix's proxy asks for the statistic. k_ns_classify: one lane per matrix adds
// the partial sums in order and writes the flag every later product reads.
struct WideRule {
  double near_lo, lo, hi;    // in units of the proxy N * ||offdiag(A0)||^2; near_lo == lo: no near range
  double near_diff;          // > 0: in the near range the gate takes a matrix whose proxy exceeds its column
                             // concentration by more than this; 0: the kColcFrac rule there as above the band
};
// kBulkShare: outlier columns keep the cheap gates while the other columns still hold a few
// thousandths of the mass (1 % of the columns x100: 1e-2 of it, 8e-4 .. 1.6e-3 with those gates);
// beyond that the bulk's directions drown in the rounding of the outliers (x300: share 1e-3, 1.4e-3
// .. 1.9e-3; x1000: 1e-4, 3.6e-3 .. 4.0e-3; x3000: 5.2e-3 .. 5.8e-3) and only every residual
// term from iteration 1 on recovers them (8e-5 .. 2.9e-4).
// kColcFrac: a matrix keeps the cheap gates only if its column norms explain its proxy (colc at least
// 0.85 of it: pure outlier columns and scaled columns read 1.00 .. 1.01). Anything less is a
// mixture (a low-rank signal WITH outlier columns: 3.5e-3 at a ratio of 0.28 and 6.6e-3 at 0.5 with
// the cheap gates at 1024x3072, 1e-4 .. 2e-4 with every residual term) or has its mass in directions
// that are not columns at all (near-duplicate rows: ratio 0.5 .. 0.75).
constexpr double kColcFrac = 0.85, kBulkShare = 3e-3;
__device__ __forceinline__ double cond_proxy(const double *c, int N) {
  double s = c[0];
#pragma unroll
  for (int i = 1; i < kCondParts; ++i) s = s + c[i];
  return s * (double)N;
}
__device__ __host__ __forceinline__ bool wants_colstat(const WideRule &r, double p) {
  return p >= r.hi || (p > r.near_lo && p <= r.lo);
}
struct NsColArgs {
  int n;
  int blocks[kMaxGroups];          // colstat: E * parts, classify: E
  const uint16_t *Xh[kMaxGroups];  // (E, M, N) row-major
  const double *cond[kMaxGroups];
  double *part[kMaxGroups];        // (E, parts, 2)
  int32_t *flag[kMaxGroups];       // (E)
  int M[kMaxGroups], N[kMaxGroups], parts[kMaxGroups];
  WideRule rule[kMaxGroups];
};
constexpr int kColBlock = 64;       // columns per block of k_ns_colstat (measured: 64 -> 92 us, 256 -> 104 us
                                    // per Qwen3-0.6B step: more blocks beat longer row pieces)
constexpr int kColLanes = kColBlock / 8, kColRowGroups = kThreads / kColLanes;
constexpr int kColRowStep = 4;      // every fourth row: the thresholds are coarse (a quarter of the proxy; 1.3
                                    // against 1.0 and 1.9+), a quarter of the rows places a matrix as well as all
                                    // of them (flat columns read 1 + 8/M more) and costs a quarter of the bytes
__global__ void __launch_bounds__(kThreads) k_ns_colstat(NsColArgs a) {
  __shared__ double colsum[kColRowGroups][kColBlock];
  __shared__ double wave_sum[2][kColBlock / 64];
  int b = (int)blockIdx.x, q = 0;
  while (q + 1 < a.n && b >= a.blocks[q]) { b -= a.blocks[q]; ++q; }
  const int e = b / a.parts[q], part = b % a.parts[q];
  const int M = a.M[q], N = a.N[q];
  if (!wants_colstat(a.rule[q], cond_proxy(a.cond[q] + (int64_t)e * kCondParts, N))) return;
  // lane (rg, cg): columns part*64 + 8*cg .. +7 (one 16-byte load per row), rows 4 rg, 4 (rg + 32), ...
  const int cg = (int)threadIdx.x % kColLanes, rg = (int)threadIdx.x / kColLanes;
  const int j = part * kColBlock + 8 * cg;
  double c[8] = {0.0, 0.0, 0.0, 0.0, 0.0, 0.0, 0.0, 0.0};
  if (j < N) {
    const uint16_t *src = a.Xh[q] + (int64_t)e * M * N + j;
#pragma unroll 8
    for (int i = kColRowStep * rg; i < M; i += kColRowStep * kColRowGroups) {
      const anc_u32x4 w = *(const anc_u32x4 *)(src + (int64_t)i * N);
      const uint32_t u[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const double x0 = (double)__uint_as_float(u[k] << 16), x1 = (double)__uint_as_float(u[k] & 0xFFFF0000u);
        c[2 * k] = c[2 * k] + x0 * x0;
        c[2 * k + 1] = c[2 * k + 1] + x1 * x1;
      }
    }
  }
#pragma unroll
  for (int k = 0; k < 8; ++k) colsum[rg][8 * cg + k] = c[k];
  __syncthreads();
  if (threadIdx.x < kColBlock) {               // one lane per column: the row groups in order
    double c2 = colsum[0][threadIdx.x];
#pragma unroll
    for (int r = 1; r < kColRowGroups; ++r) c2 = c2 + colsum[r][threadIdx.x];
    const double s2 = anc_wave_sum_f64(c2), s4 = anc_wave_sum_f64(c2 * c2);
    if ((threadIdx.x & 63) == 0) { wave_sum[0][threadIdx.x >> 6] = s2; wave_sum[1][threadIdx.x >> 6] = s4; }
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    double t2 = wave_sum[0][0], t4 = wave_sum[1][0];
#pragma unroll
    for (int w = 1; w < kColBlock / 64; ++w) { t2 = t2 + wave_sum[0][w]; t4 = t4 + wave_sum[1][w]; }
    double *out = a.part[q] + ((int64_t)e * a.parts[q] + part) * 2;
    out[0] = t2;
    out[1] = t4;
  }
}
static_assert(kColBlock % 64 == 0 && kColBlock <= kThreads, "k_ns_colstat: whole wavefronts of one lane per column in the final sum");
__global__ void __launch_bounds__(kThreads) k_ns_classify(NsColArgs a) {
  int t = (int)(blockIdx.x * kThreads + threadIdx.x), q = 0;
  while (q + 1 < a.n && t >= a.blocks[q]) { t -= a.blocks[q]; ++q; }
  if (t >= a.blocks[q]) return;
  const int e = t, N = a.N[q];
  const WideRule r = a.rule[q];
  const double p = cond_proxy(a.cond[q] + (int64_t)e * kCondParts, N);
  bool wide = p > r.lo && p < r.hi;
  if (!wide && wants_colstat(r, p)) {
    const double *c = a.part[q] + (int64_t)e * a.parts[q] * 2;
    double s2 = c[0], s4 = c[1], lightest = c[0];
    for (int i = 1; i < a.parts[q]; ++i) {
      s2 = s2 + c[2 * i];
      s4 = s4 + c[2 * i + 1];
      lightest = c[2 * i] < lightest ? c[2 * i] : lightest;
    }
    const double colc = s2 > 0.0 ? (double)N * s4 / (s2 * s2) : 1.0;
    // outlier columns: the share of the mass outside them, from the lightest block of columns
    const double bulk = s2 > 0.0 ? (double)a.parts[q] * lightest / s2 : 1.0;
    if (p < r.hi && r.near_diff > 0.0) wide = p - colc > r.near_diff;
    else wide = colc < kColcFrac * p || (p >= r.hi && bulk < kBulkShare);
  }
  a.flag[q][e] = wide ? 1 : 0;
}

// ------------------------------------------------------------------------- workspace
struct Carve {
  uint64_t base;
  int64_t off = 0;
  explicit Carve(uint64_t b) : base(b) {}
  template <typename T> T *take(int64_t count) {
    T *p = (T *)(base + (uint64_t)off);
    off += (count * (int64_t)sizeof(T) + 255) / 256 * 256;
    return p;
  }
};

// Which iterations carry bf16 residual operands. Rounding X to bf16 costs about 1e-3 of
// relative Frobenius error per late iteration on square Gaussian inputs (less on wide
// ones, more on small ones); measured against the fp32 numpy chain, 5 Polar-Express steps:
//   no residuals         1024x1024 2.2e-3   1024x2048 1.4e-3   1024x3072 1.2e-3   256x256 2.8e-3
//   X in the last two    1024x1024 1.4e-3                                         256x256 2.4e-3
//   X, F, B in last three 1024x1024 7e-5                                          256x256 3e-4
// The plan depends on (M, N, steps) only, never on the batch.
struct SplitPlan {
  int x_from;    // first iteration whose A and B X products add the residual of X for every matrix
  int fb_from;   // first iteration whose A A and B X products add the residuals of F and Boff
  // Conditioning gates. In iteration k < x_from with gate_tau[k] > 0, a matrix whose proxy
  // N * ||offdiag(A0)||_F^2 exceeds gate_tau[k] adds the residual of X to A = X X^T and, with bit k
  // of gate_bx set, to X = a X + B X as well.
  static constexpr int kGateIters = 8;
  float gate_tau[kGateIters];
  unsigned gate_bx;
  // The wide gate: a matrix whose proxy lies in (wide_lo, wide_hi), or outside it with a column
  // statistic that says so (k_ns_classify), adds the residual of X to A = X X^T from iteration
  // wide_gram_from on and the residuals of X, F and Boff to all three products from iteration
  // wide_all_from on. wide_hi == 0: no such gate.
  float wide_lo, wide_hi, wide_near;   // wide_near: start of the near range below the band (== wide_lo: none)
  float wide_near_diff;                // see WideRule::near_diff
  int wide_gram_from, wide_all_from;
  // No fp32 copy of A except for the matrices the wide gate flags: B = b A + c A A takes the
  // off-diagonal entries of A from the bf16 Fh it multiplies anyway. Costs 3 .. 8 % of accuracy where
  // N >= 2M (independent entries 1.36e-3 -> 1.41e-3 at 1024x2048 and 1.16e-3 -> 1.20e-3 at 1024x3072,
  // 1 % of the columns x100 1.58e-3 -> 1.66e-3 and 1.15e-3 -> 1.24e-3) and saves 6 of the 13 bytes
  // per element of A an iteration moves; N < 2M keeps the copy (the column-scaled probe input at
  // 1024x1024 would go from 1.85e-3 to 2.10e-3).
  bool drop_a32;
  // The low half of the iterate as one byte per element wherever it is never a matrix-core operand
  // (NsGemm::l8_in): the matrices that take no gate, and for a gated one every iterate but those its
  // gated products read. 3 instead of 4 bytes per element read and written by X = a X + B X; the
  // numpy model of this chain puts the cost at the fourth digit (1.4077e-3 -> 1.4074e-3 at
  // 1024x2048, 1.1997e-3 -> 1.1985e-3 at 1024x3072). The result itself moves by 1.2e-3: the chain
  // turns any perturbation of its iterate, this one of 2^-16 per element included, into another
  // realisation of its own rounding error (an exact low half moves it as far). Measured: X = a X +
  // B X 4.85 -> 4.69 ms per step of Qwen3-0.6B, 2.0 GB less HBM traffic.
  bool low8;
  bool gated(int k) const { return k >= 0 && k < kGateIters && k < x_from && gate_tau[k] > 0.0f; }
  bool wide() const { return wide_hi > 0.0f; }
  bool wide_gram(int k) const { return wide() && k >= wide_gram_from && k < x_from; }
  bool wide_all(int k) const { return wide() && k >= wide_all_from && k < fb_from; }
  bool any_gate(int steps) const {
    if (wide()) return true;
    for (int k = 0; k < steps; ++k) if (gated(k)) return true;
    return false;
  }
};
// The proxy is 1.0 for a matrix with independent entries whatever its row scaling (1.2 with 1 %
// of the rows x100), 1.7 for columns scaled over 0.1..3, about 100 with 1 % of the columns x100.
//   kTauHard: inputs whose Frobenius mass sits in a few directions spread over all rows (a
//     gradient with a few outlier columns: the transposed iterate of a tall weight with outlier
//     rows). Rounding X to bf16 then costs the small directions their signal in A = X X^T while the
//     large ones converge: 1% of the columns x100 gives 2.2e-3 at 1024x3072 and 3.8e-3 at
//     1024x1024 without the extra terms of iterations 1-2, 1.2e-3 and 8e-4 with them. Row outliers,
//     whose mass lands on the exact fp32 diagonal of A, need nothing (5e-4 .. 7e-4).
//   kTauPlain: N < 2M runs the residual of X in both X-products of the last two iterations; a
//     matrix with independent entries needs them in the last one only (1.66e-3 against 1.41e-3 at
//     1024x1024, 5.3e-4 either way with outlier rows), the column-scaled case needs both (1.85e-3
//     against 2.09e-3). So the first of the two is gated low. Between the two thresholds square
//     matrices were still within 4 % of the bar (columns scaled over 0.03..3, proxy 1.79: 1.93e-3;
//     log-normal column scales, sigma 0.45, proxy 2.2: 1.79e-3), so iteration 2 carries the same
//     two terms behind the same gate: 1.48e-3 and 1.25e-3.
//   kTauWideLo .. kTauWideHi: inputs whose spectrum is spread over decades, or with many moderately
//     large columns. Measured proxies (1024x1024 / 1024x3072): log-uniform spectrum over one decade
//     1.4 / 4.0, 1.5 decades 2.4 / 7.4, two 3.6 / 11.3, three 5.8 / 19.4; 10 % of the columns x10 8.4;
//     against 1 % of the columns x100 100, x1000 102, a rank-32 signal over noise 32 / 95, a
//     power-law spectrum 146 / 437. In the band the plan above leaves 2.5e-3 .. 4.2e-3 (every operand
//     rounding of the later iterations counts: the small singular values are still far from 1);
//     with all residuals in all products from iteration 2 on 1.0e-4 .. 4.8e-4, from iteration 1 on
//     (what runs) 2e-5 .. 8e-5. Above the band the gates above suffice for outlier columns (8e-4 ..
//     1.4e-3; only outliers x1000 miss the bar, with or without these terms at 1024x1024).
//   Outside the band the column statistic decides (k_ns_colstat): a matrix whose column
//     concentration explains less than kColcFrac of its proxy is not a matrix of outlier or scaled
//     columns. Above the band that is a low-rank signal over weak noise or a steep spectrum, alone
//     or mixed with outlier columns (rank 32 + 10 % noise at 1024x2048 / 1024x3072, proxy 65 / 97:
//     2.9e-3 with the gates above, 1.4e-4 with the wide gate's terms; + 1 % noise 5.0e-3 -> 2.5e-4);
//     just below it (kTauWideNear .. kTauWideLo, N < 2M only) a gap in the spectrum with flat
//     column norms (a fraction of near-duplicate rows: proxy 1.55 / 1.7 / 1.8 / 2.0 gives 1.44e-3 /
//     1.74e-3 / 1.98e-3 / 2.4e-3 with the low gate, 3e-5 .. 5e-5 with these terms), while scaled
//     columns (concentration = proxy) stay with the low gate.
//   The wide gate's terms start at iteration 1: from iteration 2 the low-rank cases above stay at
//     1.5e-3 .. 2.7e-3.
//   N >= 2M carries no residual term in its plan and has no low gate: an input whose spectrum has
//     a gap with flat column norms (a fraction of near-duplicate rows, proxy 1 + twice that fraction
//     times N/M) would leave the bar between proxy 1.2 and the band: 1024x2048 reads 1.80e-3 at
//     proxy 1.15, 2.15e-3 at 1.3, 2.8e-3 at 1.6, 4.6e-3 at 2.3 (1024x3072: 1.57e-3, 1.91e-3, 2.5e-3,
//     3.7e-3) with the plan alone. What decides is the part of the proxy the column norms do not
//     explain: with the columns of such a matrix scaled by exp(sigma z), sigma 0 .. 0.4 (proxy up to
//     2.5), the error stays a function of proxy - colc alone (0.10: 1.67e-3 .. 1.76e-3, 0.19: 1.90e-3
//     .. 1.94e-3, 0.29: 2.12e-3 .. 2.15e-3, 0.5: 2.5e-3 .. 2.6e-3 at 1024x2048), where the ratio
//     colc / proxy moves from 0.78 to 0.87. So the near range of these shapes starts at
//     kTauWideNear2M and takes a matrix with proxy - colc > kNearDiff2M (the wide gate's terms: 1e-5
//     .. 5e-5). Independent entries, outlier rows, scaled or outlier columns and heavy tails read
//     proxy - colc < 0.01. (A cheaper gate for the range -- the residual of X in both X-products of
//     iterations 2 .. 4, 6e-4 .. 1.4e-3 in the numpy model of this chain -- was built and taken out
//     again: a GPU fault in the test run that carried it, cause not found.)
constexpr float kTauWideNear2M = 1.15f, kNearDiff2M = 0.15f;
constexpr float kTauHard = 2.5f, kTauPlain = 1.3f, kTauWideLo = 2.5f, kTauWideHi = 40.0f, kTauWideNear = 1.5f;
SplitPlan split_plan(int64_t M, int64_t N, int mode, int steps) {
  SplitPlan sp{};
  sp.x_from = sp.fb_from = steps;
  if (mode == ANC_NS_BF16_X3) {
    // every product with the residuals of both operands' bf16 roundings, in every iteration:
    // about 1e-5 on every input tried, three times the matrix-core work
    sp.x_from = sp.fb_from = 0;
    return sp;
  }
  if (mode == ANC_NS_BF16_LATE3 && M >= 1024) {
    // For coefficients that do not drive the singular values to 1 (Keller's quintic leaves them in
    // 0.7 .. 1.2, so offdiag(A) never becomes small and every operand rounding stays first-order:
    // the gated plan below gives 3.7e-3 at 1024x1024 and 2.8e-3 at 1024x3072 there). Every matrix,
    // no gates of its own: the residual of X from iteration 2 on, those of F and Boff from
    // iteration 3 on. All three from iteration 2: 6e-5 / 3e-5 for 2.2 times the plain chain; all
    // three in the last two iterations only: 2.2e-3 at 1024x1024. M < 1024 runs a heavier plan
    // in either mode (below).
    // From a fixed iteration on whatever the chain's length (Keller's iterates do not settle, so a
    // longer chain keeps adding first-order roundings: with the last three iterations only, 6 steps
    // gave 3.1e-3 and 8 steps 8.9e-3 at 1024x1024), and the last three of a shorter one.
    sp.x_from = sp.fb_from = steps >= 5 ? 2 : (steps > 3 ? steps - 3 : 0);
    // The residuals of F and Boff can start one iteration after that of X: 8e-4 at 1024x1024
    // (independent entries, scaled columns, outlier columns alike) and 4e-4 .. 7.5e-4 at 1024x3072
    // for 2.05 instead of 2.2 times the plain chain's work. (F and Boff first and X later, or the
    // last two iterations only: 2.0e-3 .. 2.3e-3.)
    if (steps >= 5) sp.fb_from = sp.x_from + 1;
    // and the matrices the wide gate flags (below) start one iteration earlier, as they do under
    // Polar Express: a rank-32 signal over 1 % noise is 2.1e-3 at 1024x1024 with the terms from
    // iteration 2 and 3e-4 from iteration 1
    if (sp.x_from > 1) {
      sp.wide_lo = kTauWideLo; sp.wide_hi = kTauWideHi;
      sp.wide_near = N < 2 * M ? kTauWideNear : kTauWideLo;
      sp.wide_gram_from = 1; sp.wide_all_from = 1;
    }
    return sp;
  }
  if (mode != ANC_NS_BF16 && mode != ANC_NS_BF16_LATE3) return sp;
  // The first iterations are insensitive (the singular values are still far below 1, so
  // B X is a small correction to a X); residuals start at a fixed iteration index.
  if (M >= 1024) {
    sp.drop_a32 = mode == ANC_NS_BF16 && N >= 2 * M;
    sp.low8 = sp.drop_a32;
    if (steps >= 2) {                         // terms from iteration 1 to the end, whatever the length
                                              // (cond 1e3 without: 6 steps 4.4e-3 .. 7e-3, 8 steps 6e-3 .. 1.8e-2)
      sp.wide_lo = kTauWideLo; sp.wide_hi = kTauWideHi;
      sp.wide_near = N < 2 * M ? kTauWideNear : kTauWideLo;
      if (mode == ANC_NS_BF16 && N >= 2 * M) { sp.wide_near = kTauWideNear2M; sp.wide_near_diff = kNearDiff2M; }
      sp.wide_gram_from = 1; sp.wide_all_from = 1;
    }
    if (N < 2 * M) {
      sp.x_from = steps - 2 < 3 ? steps - 2 : 3;
      sp.gate_tau[1] = sp.gate_tau[2] = kTauHard;
      if (steps == 5) {                       // the schedule the low gate was measured on
        sp.gate_tau[2] = sp.gate_tau[3] = kTauPlain;
        sp.gate_bx = (1u << 2) | (1u << 3);
        sp.x_from = 4;
      }
    } else {
      // N >= 2M: iteration 2 alone (1 % of the columns x100 without it: 1024x2048 1.6e-3 .. 1.7e-3,
      // 1024x2560 1.8e-3, 1536x3072 2.1e-3, 1024x3072 2.2e-3, 2048x4096 2.2e-3, 4096x8192 2.3e-3;
      // with it 1.0e-3 .. 1.2e-3). One rule for every such shape.
      sp.gate_tau[2] = kTauHard;
      // a chain shorter than the 5 steps this was measured on ends before iteration 2's term has
      // paid off (3 steps at 1024x3072: 2.3e-3, 2 steps 2.7e-3): iteration 1 as well
      if (steps < 5) sp.gate_tau[1] = kTauHard;
    }
  } else {
    // Small matrices average fewer rounding errors per element and cost next to nothing: all
    // residuals from iteration 1 on, from iteration 0 below M = 256, no gates. With them from
    // iteration 2 (relative Frobenius error, Polar Express / Keller): 128x128 condition number 1e3
    // 4.0e-3 / 2.8e-3, columns scaled 0.1..3 under Keller 2.5e-3, 128x384 and 256x512 condition
    // number 1e3 5.5e-3 / 4.0e-3 and 2.4e-3 / 1.8e-3, 512x1024 with 1 % of the columns x100
    // 4.4e-3; from iteration 1: at most 1.0e-3 on all of these from M = 256 on; 128x128 with one
    // column x100 still 4.8e-3, 1e-5 from iteration 0.
    const int from = M < 256 ? 0 : 1;
    sp.x_from = sp.fb_from = steps - 3 < from ? steps - 3 : from;
  }
  if (sp.x_from < 0) sp.x_from = 0;
  if (sp.fb_from < 0) sp.fb_from = 0;
  return sp;
}

struct Plan {
  int nchunks;
  bool split;
  SplitPlan sp;
  uint16_t *Fl, *Bl;
  double *partials;
  float *recip;
  float *pow2;           // (E) power-of-two pre-scale of tiny inputs, pair entries
  double *cond;          // (E, kCondParts) conditioning proxy, bf16 modes
  double *colpart;       // (E, col_parts, 2) column statistic, plans with a wide gate
  int32_t *wide_flag;    // (E) the wide gate's decision
  int col_parts;
  // bf16 modes
  uint16_t *Xh[2], *Xl[2];
  float *A32, *dA, *dB;
  uint16_t *Fh, *Bh;
  // fp32 mode
  float *Af, *Bf, *Yf;
  int64_t bytes;
};

Plan make_plan(uint64_t base, int64_t E, int64_t M, int64_t N, int mode, int steps) {
  Plan pl{};
  Carve c(base);
  pl.nchunks = (int)((M * N + ANC_GN_CHUNK - 1) / ANC_GN_CHUNK);
  pl.sp = split_plan(M, N, mode, steps);
  pl.split = pl.sp.x_from < steps;
  pl.partials = c.take<double>(E * pl.nchunks);
  pl.recip = c.take<float>(E);
  pl.pow2 = c.take<float>(E);
  if (mode == ANC_NS_FP32) {
    pl.Af = c.take<float>(E * M * M);
    pl.Bf = c.take<float>(E * M * M);
    pl.Yf = c.take<float>(E * M * N);
  } else {
    for (int i = 0; i < 2; ++i) {
      pl.Xh[i] = c.take<uint16_t>(E * M * N);
      pl.Xl[i] = c.take<uint16_t>(E * M * N);
    }
    pl.A32 = c.take<float>(E * M * M);
    pl.Fh = c.take<uint16_t>(E * M * M);
    pl.Bh = c.take<uint16_t>(E * M * M);
    if (pl.sp.fb_from < steps || pl.sp.wide()) {
      pl.Fl = c.take<uint16_t>(E * M * M);
      pl.Bl = c.take<uint16_t>(E * M * M);
    }
    pl.dA = c.take<float>(E * M);
    pl.dB = c.take<float>(E * M);
    pl.cond = c.take<double>(E * kCondParts);
    if (pl.sp.wide()) {
      pl.col_parts = (int)((N + kColBlock - 1) / kColBlock);
      pl.colpart = c.take<double>(E * pl.col_parts * 2);
      pl.wide_flag = c.take<int32_t>(E);
    }
  }
  pl.bytes = c.off;
  return pl;
}

int check_shape(int64_t E, int64_t M, int64_t N, int mode, const char *who) {
  ANC_REQUIRE(E > 0 && M > 0 && N > 0, "%s: E, M, N must be positive", who);
  ANC_REQUIRE(M % 128 == 0 && N % 128 == 0, "%s: (M,N)=(%lld,%lld) must be multiples of 128", who,
              (long long)M, (long long)N);
  ANC_REQUIRE(M <= N, "%s: M=%lld > N=%lld; pass tall matrices transposed", who, (long long)M,
              (long long)N);
  ANC_REQUIRE(mode == ANC_NS_BF16 || mode == ANC_NS_FP32 || mode == ANC_NS_BF16_FAST || mode == ANC_NS_BF16_X3 ||
                  mode == ANC_NS_BF16_LATE3,
              "%s: unknown mode %d", who, mode);
  ANC_REQUIRE(E * (M / 128) * (N / 128) < (1ll << 30) && E * M * N < (1ll << 40),
              "%s: batch too large", who);
  return ANC_OK;
}

// One problem of a chain launch: a batch of E (M,N) matrices with its workspace plan.
struct ChainProb {
  Plan pl;
  const uint16_t *inH, *inL;   // the input bf16 pair
  int nxt;                     // which pair of the plan receives the first step's output
  const float *scale0;         // per-matrix factor the first step applies to its input, or null
  float *X32;                  // fp32 result (may overlay the input pair when steps >= 2)
  int64_t E, M, N;
  const anc_muon_desc_t *upd;  // or: the weights (E entries) the last step updates in its epilogue
};

// steps x { A = X X^T; B = b A + c A A; X = a X + B X } on n problems side by side: every
// product of a step is ONE launch over all problems (problems in the order given; put the
// longest K first). First step's output goes to pair `nxt` of each plan, later steps ping-pong;
// the last step writes the fp32 results. With n == 1 and a shape that is not a multiple of 256
// (or force_small) the 128x128-tile kernel runs instead.
int run_bf16_chain(ChainProb *cp, int n, int steps, const float *coef, bool force_small, hipStream_t s,
                   const NsUpdate *upd = nullptr) {
  bool big = !force_small;
  for (int q = 0; q < n; ++q) big = big && (cp[q].M % 256 == 0) && (cp[q].N % 256 == 0);
  ANC_REQUIRE(big || n == 1, "Newton-Schulz chain: several problems per launch need dims that are multiples of 256");
  const uint16_t *curH[kMaxGroups], *curL[kMaxGroups];
  int nxt[kMaxGroups];
  int64_t Es[kMaxGroups];
  for (int q = 0; q < n; ++q) { curH[q] = cp[q].inH; curL[q] = cp[q].inL; nxt[q] = cp[q].nxt; Es[q] = cp[q].E; }
  bool want_cond = false;      // some later iteration gates a product on the proxy
  for (int q = 0; q < n; ++q) want_cond = want_cond || cp[q].pl.sp.any_gate(steps);
  double l8_cur[kMaxGroups];   // the proxy bound the current iterate's 8-bit low halves were written with (0: none)
  for (int q = 0; q < n; ++q) l8_cur[q] = 0.0;
  for (int k = 0; k < steps; ++k) {
    const bool last = k + 1 == steps;
    NsGemm ga[kMaxGroups], gb[kMaxGroups], gx[kMaxGroups];
    for (int q = 0; q < n; ++q) {
      const Plan &pl = cp[q].pl;
      const int64_t M = cp[q].M, N = cp[q].N, mn = M * N;
      const bool split = k >= pl.sp.x_from;        // X residual terms
      const bool split_fb = k >= pl.sp.fb_from;    // F and Boff residual terms
      const int tile = big ? 256 : BM;
      const int tM = (int)(M / tile), tN = (int)(N / tile);
      NsGemm g{};
      g.M = (int)M; g.N = (int)N;
      g.A32 = pl.A32; g.Fh = pl.Fh; g.dA = pl.dA; g.Bh = pl.Bh; g.dB = pl.dB;
      if (pl.sp.drop_a32) {
        // the first iteration runs before the classification: nobody is flagged yet
        g.a32_gated = 1;
        g.a32_flag = (k > 0 && pl.sp.wide()) ? pl.wide_flag : nullptr;
      }
      g.Fl = split_fb ? pl.Fl : nullptr;
      g.Bl = split_fb ? pl.Bl : nullptr;
      g.ca = coef[3 * k]; g.cb = coef[3 * k + 1]; g.cc = coef[3 * k + 2];
      g.scale = (k == 0) ? cp[q].scale0 : nullptr;
      // 256-tile kernels: everything the chain itself writes (F, B, every iterate after the input)
      // is in panel layout; the input pair is row-major as the caller left it
      g.f_panel = big ? 1 : 0;
      g.x_panel = (big && k > 0) ? 1 : 0;
      g.y_panel = big ? 1 : 0;
      // the wide gate of this iteration (a band of the proxy; the proxy is N * sum, hence the / N)
      const bool wide_g = pl.sp.wide_gram(k);      // implies !split
      const bool wide_a = pl.sp.wide_all(k);       // implies !split_fb
      auto set_wide = [&](NsGemm &w, int nterms_wide) {
        w.wide_flag = pl.wide_flag;
        w.nterms_wide = nterms_wide;
      };
      // A = X X^T
      ga[q] = g;
      ga[q].A[0] = curH[q]; ga[q].B[0] = curH[q]; ga[q].nterms = 1;
      const bool gated = pl.sp.gated(k);           // implies !split
      if (split || gated || wide_g) {
        ga[q].A[1] = curH[q]; ga[q].B[1] = curL[q];
        ga[q].A[2] = curL[q]; ga[q].B[2] = curH[q];
        if (split) ga[q].nterms = 3;
      }
      if (gated) {
        ga[q].cond = pl.cond;
        ga[q].cond_thresh = (double)pl.sp.gate_tau[k] / (double)N;
        ga[q].nterms_hard = 3;
      }
      if (wide_g) set_wide(ga[q], 3);
      if (wide_a) {                                // the residual of F, for the matrices in the band only
        set_wide(ga[q], split ? 0 : 3);
        ga[q].Fl = pl.Fl;
        ga[q].lo_gated = 1;
      }
      ga[q].K = (int)N; ga[q].strideA = mn; ga[q].strideB = mn; ga[q].tiles_m = tM; ga[q].tiles_n = tM; ga[q].lower = 1;
      // B = b A + c A A
      gb[q] = g;
      gb[q].A[0] = pl.Fh; gb[q].B[0] = pl.Fh; gb[q].nterms = 1;
      if (split_fb || wide_a) {
        gb[q].A[1] = pl.Fh; gb[q].B[1] = pl.Fl;
        gb[q].A[2] = pl.Fl; gb[q].B[2] = pl.Fh;
        if (split_fb) gb[q].nterms = 3;
      }
      if (wide_a) {
        set_wide(gb[q], 3);
        gb[q].Bl = pl.Bl;
        gb[q].lo_gated = 1;
      }
      gb[q].K = (int)M; gb[q].strideA = M * M; gb[q].strideB = M * M; gb[q].tiles_m = tM; gb[q].tiles_n = tM; gb[q].lower = 1;
      // X = a X + B X
      gx[q] = g;
      gx[q].A[0] = pl.Bh; gx[q].B[0] = curH[q]; gx[q].nterms = 1;
      if (split) { gx[q].A[gx[q].nterms] = pl.Bh; gx[q].B[gx[q].nterms] = curL[q]; ++gx[q].nterms; }
      if (gated && ((pl.sp.gate_bx >> k) & 1u) && !split_fb) {
        gx[q].A[1] = pl.Bh; gx[q].B[1] = curL[q];
        gx[q].cond = pl.cond;
        gx[q].cond_thresh = (double)pl.sp.gate_tau[k] / (double)N;
        gx[q].nterms_hard = 2;
      }
      if (split_fb) { gx[q].A[gx[q].nterms] = pl.Bl; gx[q].B[gx[q].nterms] = curH[q]; ++gx[q].nterms; }
      if (wide_a) {                                // [Bh Xh, Bh Xl, Bl Xh]: the lists above are prefixes of it
        gx[q].A[1] = pl.Bh; gx[q].B[1] = curL[q];
        gx[q].A[2] = pl.Bl; gx[q].B[2] = curH[q];
        set_wide(gx[q], 3);
      }
      gx[q].K = (int)M; gx[q].strideA = M * M; gx[q].strideB = mn; gx[q].tiles_m = tM; gx[q].tiles_n = tN; gx[q].lower = 0;
      gx[q].Xh = curH[q]; gx[q].Xl = curL[q];
      gx[q].Yh = last ? nullptr : pl.Xh[nxt[q]];
      gx[q].Yl = last ? nullptr : pl.Xl[nxt[q]];
      gx[q].X32 = (last && cp[q].upd == nullptr) ? cp[q].X32 : nullptr;
      gx[q].upd = last ? cp[q].upd : nullptr;
      // The next iterate's low half is one byte for the matrices whose low half no product of the
      // next iteration multiplies: every matrix outside the wide gate if that iteration has no gate,
      // those below its gate if it has one, none if its plan splits X for everybody.
      double l8_next = 0.0;
      if (big && pl.sp.low8 && !last && pl.sp.any_gate(steps) && k + 1 < pl.sp.x_from)
        l8_next = pl.sp.gated(k + 1) ? (double)pl.sp.gate_tau[k + 1] / (double)N : 1e300;
      gx[q].l8_cond = pl.cond;
      gx[q].l8_wide = pl.sp.wide() ? pl.wide_flag : nullptr;
      gx[q].l8_in = l8_cur[q];
      gx[q].l8_out = l8_next;
      l8_cur[q] = l8_next;
    }
    const int tM0 = (int)(cp[0].M / BM), tN0 = (int)(cp[0].N / BN);
    const unsigned g_sym = (unsigned)(cp[0].E * tM0 * (tM0 + 1) / 2), g_mn = (unsigned)(cp[0].E * tM0 * tN0);
    {
      AncProfScope prof(ANC_PROF_NS_GRAM, s);
      if (big) { if (int rc = anc_ns_gemm_big_multi(EPI_GRAM, ga, Es, n, s)) return rc; }
      else hipLaunchKernelGGL(k_ns_gemm<EPI_GRAM>, dim3(g_sym), dim3(kGemmThreads), 0, s, ga[0]);
    }
    ANC_LAUNCH_CHECK();
    if (k == 0 && want_cond) {
      // the proxy of every problem that gates a later product, from the Fh this launch wrote
      NsCondArgs ca{};
      int blocks = 0;
      for (int q = 0; q < n; ++q) {
        if (!cp[q].pl.sp.any_gate(steps)) continue;
        ca.Fh[ca.n] = cp[q].pl.Fh; ca.out[ca.n] = cp[q].pl.cond; ca.M[ca.n] = (int)cp[q].M;
        ca.blocks[ca.n] = (int)(cp[q].E * kCondParts);
        blocks += ca.blocks[ca.n];
        ++ca.n;
      }
      AncProfScope prof(ANC_PROF_NS_FRO, s);
      hipLaunchKernelGGL(k_ns_cond, dim3((unsigned)blocks), dim3(kThreads), 0, s, ca);
      ANC_LAUNCH_CHECK();
      // the wide gate's decision per matrix, from the proxy and, where it asks, the column norms
      NsColArgs cs{}, cf{};
      int cs_blocks = 0, cf_lanes = 0;
      for (int q = 0; q < n; ++q) {
        const Plan &pl = cp[q].pl;
        if (!pl.sp.wide()) continue;
        const int i = cs.n;
        cs.Xh[i] = cp[q].inH; cs.cond[i] = pl.cond; cs.part[i] = pl.colpart; cs.flag[i] = pl.wide_flag;
        cs.M[i] = (int)cp[q].M; cs.N[i] = (int)cp[q].N; cs.parts[i] = pl.col_parts;
        cs.rule[i] = WideRule{(double)pl.sp.wide_near, (double)pl.sp.wide_lo, (double)pl.sp.wide_hi,
                              (double)pl.sp.wide_near_diff};
        cs.blocks[i] = (int)(cp[q].E * pl.col_parts);
        cs_blocks += cs.blocks[i];
        ++cs.n;
      }
      if (cs.n > 0) {
        cf = cs;
        for (int i = 0; i < cf.n; ++i) { cf.blocks[i] = cs.blocks[i] / cs.parts[i]; cf_lanes += cf.blocks[i]; }
        hipLaunchKernelGGL(k_ns_colstat, dim3((unsigned)cs_blocks), dim3(kThreads), 0, s, cs);
        ANC_LAUNCH_CHECK();
        hipLaunchKernelGGL(k_ns_classify, dim3((unsigned)((cf_lanes + kThreads - 1) / kThreads)), dim3(kThreads), 0, s, cf);
        ANC_LAUNCH_CHECK();
      }
    }
    {
      AncProfScope prof(ANC_PROF_NS_BMAT, s);
      if (big) { if (int rc = anc_ns_gemm_big_multi(EPI_BMAT, gb, Es, n, s)) return rc; }
      else hipLaunchKernelGGL(k_ns_gemm<EPI_BMAT>, dim3(g_sym), dim3(kGemmThreads), 0, s, gb[0]);
    }
    ANC_LAUNCH_CHECK();
    {
      AncProfScope prof(last && upd != nullptr ? ANC_PROF_NS_BX_UPD : ANC_PROF_NS_BX, s);
      if (big) { if (int rc = anc_ns_gemm_big_multi(EPI_BX, gx, Es, n, s, last ? upd : nullptr)) return rc; }
      else hipLaunchKernelGGL(k_ns_gemm<EPI_BX>, dim3(g_mn), dim3(kGemmThreads), 0, s, gx[0]);
    }
    ANC_LAUNCH_CHECK();
    for (int q = 0; q < n; ++q) {
      curH[q] = cp[q].pl.Xh[nxt[q]]; curL[q] = cp[q].pl.Xl[nxt[q]];
      nxt[q] ^= 1;
    }
  }
  return ANC_OK;
}

}  // namespace

extern "C" int64_t anc_ns_workspace_bytes(int64_t E, int64_t M, int64_t N, int mode) {
  mode &= ~ANC_NS_TILE128;
  if (check_shape(E, M, N, mode, "anc_ns_workspace_bytes")) return -1;
  // sized for any step count: with steps >= 3 every optional buffer of the mode's plan is present
  // (the longer of a long and a 5-step chain's plans, should the two ever differ)
  const int64_t a = make_plan(0, E, M, N, mode, 64).bytes, b = make_plan(0, E, M, N, mode, 5).bytes;
  return a > b ? a : b;
}

// FLOPs of the output tiles a symmetric M x M product really multiplies, per unit of K: the tiles
// on or below the diagonal, 256x256 where the 256-tile kernel runs (dims multiples of 256 and the
// 128-tile kernel not forced), else 128x128. A diagonal tile is multiplied in full, so the count is
// 10/16 of the dense product at M = 1024 with 256-tiles and 36/64 with 128-tiles; the matrix-
// instruction counter of the profiler reads exactly this.
static double sym_tile_flops(int64_t M, int64_t N, bool force_small) {
  const double ts = (!force_small && M % 256 == 0 && N % 256 == 0) ? 256.0 : 128.0;
  const double t = (double)M / ts;
  return t * (t + 1) / 2 * 2.0 * ts * ts;
}

// Matrix-core work of one chain call: `executed` counts the tiles and terms actually
// multiplied (symmetric products compute the lower tiles only; residual terms count),
// `dense` is the textbook steps*(4 M^2 N + 2 M^3) per matrix.
extern "C" int anc_ns_flops(int64_t E, int64_t M, int64_t N, int steps, int mode,
                            double *executed, double *dense) {
  const bool force_small = (mode & ANC_NS_TILE128) != 0;
  mode &= ~ANC_NS_TILE128;
  if (int rc = check_shape(E, M, N, mode, "anc_ns_flops")) return rc;
  ANC_REQUIRE(executed != nullptr && dense != nullptr && steps >= 0, "anc_ns_flops: bad arguments");
  const double m = (double)M, n = (double)N, e = (double)E;
  *dense = e * steps * (4.0 * m * m * n + 2.0 * m * m * m);
  if (mode == ANC_NS_FP32) { *executed = *dense; return ANC_OK; }
  const SplitPlan sp = split_plan(M, N, mode, steps);
  const double sym = sym_tile_flops(M, N, force_small);
  double ex = 0.0;
  for (int k = 0; k < steps; ++k) {
    const bool sx = k >= sp.x_from, sfb = k >= sp.fb_from;
    ex += sym * (sx ? 3 : 1) * n;                                        // A = X X^T
    ex += sym * (sfb ? 3 : 1) * m;                                       // B = b A + c A A
    ex += 2.0 * m * n * (1 + (sx ? 1 : 0) + (sfb ? 1 : 0)) * m;          // X = a X + B X
  }
  *executed = e * ex;
  return ANC_OK;
}

extern "C" int anc_ns_product_flops(int64_t E, int64_t M, int64_t N, int steps, int mode, int k, int product,
                                    double *executed) {
  const bool force_small = (mode & ANC_NS_TILE128) != 0;
  mode &= ~ANC_NS_TILE128;
  if (int rc = check_shape(E, M, N, mode, "anc_ns_product_flops")) return rc;
  ANC_REQUIRE(executed != nullptr && steps > 0 && k >= 0 && k < steps && product >= 0 && product <= 2,
              "anc_ns_product_flops: bad arguments");
  const double m = (double)M, n = (double)N;
  if (mode == ANC_NS_FP32) {
    *executed = (double)E * (product == 1 ? 2.0 * m * m * m : 2.0 * m * m * n);
    return ANC_OK;
  }
  const SplitPlan sp = split_plan(M, N, mode, steps);
  const bool sx = k >= sp.x_from, sfb = k >= sp.fb_from;
  const double sym = sym_tile_flops(M, N, force_small);
  double ex;
  if (product == 0)      ex = sym * (sx ? 3 : 1) * n;
  else if (product == 1) ex = sym * (sfb ? 3 : 1) * m;
  else                   ex = 2.0 * m * n * (1 + (sx ? 1 : 0) + (sfb ? 1 : 0)) * m;
  *executed = (double)E * ex;
  return ANC_OK;
}

// Of the last chain call on this workspace: how many matrices took extra terms through a
// conditioning gate, and the matrix-core work all of them together add to anc_ns_flops' `executed`.
// Synchronises `stream`, then reads the proxy's partial sums back and takes the kernels' decisions.
extern "C" int anc_ns_hard_info(uint64_t workspace, int64_t E, int64_t M, int64_t N, int mode, int steps,
                                int32_t *n_gated, double *extra_flops, uint64_t stream) {
  const bool force_small = (mode & ANC_NS_TILE128) != 0;
  mode &= ~ANC_NS_TILE128;
  if (int rc = check_shape(E, M, N, mode, "anc_ns_hard_info")) return rc;
  ANC_REQUIRE(n_gated != nullptr && extra_flops != nullptr && workspace != 0 && steps >= 0,
              "anc_ns_hard_info: bad arguments");
  *n_gated = 0;
  *extra_flops = 0.0;
  if (mode == ANC_NS_FP32) return ANC_OK;
  const Plan pl = make_plan(workspace, E, M, N, mode, steps);
  if (!pl.sp.any_gate(steps)) return ANC_OK;
  std::vector<double> host((size_t)(E * kCondParts));
  ANC_HIP(hipStreamSynchronize(anc_stream(stream)));
  ANC_HIP(hipMemcpy(host.data(), pl.cond, host.size() * sizeof(double), hipMemcpyDeviceToHost));
  std::vector<int32_t> flags((size_t)E, 0);
  if (pl.sp.wide())
    ANC_HIP(hipMemcpy(flags.data(), pl.wide_flag, flags.size() * sizeof(int32_t), hipMemcpyDeviceToHost));
  const double gram_extra = 2.0 * sym_tile_flops(M, N, force_small) * (double)N;     // two more terms
  const double bx_extra = 2.0 * (double)M * (double)M * (double)N;                   // one more term
  for (int64_t e = 0; e < E; ++e) {
    double t = host[(size_t)(e * kCondParts)];
    for (int i = 1; i < kCondParts; ++i) t = t + host[(size_t)(e * kCondParts + i)];
    bool any = false;
    const bool in_band = flags[(size_t)e] != 0;
    for (int k = 0; k < steps; ++k) {
      if (in_band) {                    // the wide gate takes precedence over the others
        const bool sx = k >= pl.sp.x_from;
        if (pl.sp.wide_gram(k)) { *extra_flops += gram_extra; any = true; }
        if (pl.sp.wide_all(k)) {
          *extra_flops += 2.0 * sym_tile_flops(M, N, force_small) * (double)M + (sx ? 1.0 : 2.0) * bx_extra;
          any = true;
        }
        continue;
      }
      if (!pl.sp.gated(k) || !(t > (double)pl.sp.gate_tau[k] / (double)N)) continue;
      any = true;
      *extra_flops += gram_extra + (((pl.sp.gate_bx >> k) & 1u) ? bx_extra : 0.0);
    }
    if (any) ++*n_gated;
  }
  return ANC_OK;
}

extern "C" int anc_ns_batched(uint64_t X, int64_t E, int64_t M, int64_t N, int steps,
                              const float *coef, float eps, int mode, uint64_t workspace,
                              int64_t workspace_bytes, uint64_t stream) {
  const bool force_small = (mode & ANC_NS_TILE128) != 0;
  mode &= ~ANC_NS_TILE128;
  if (int rc = check_shape(E, M, N, mode, "anc_ns_batched")) return rc;
  ANC_REQUIRE(X != 0 && (X & 15) == 0, "anc_ns_batched: X must be a 16-byte aligned device pointer");
  ANC_REQUIRE(steps >= 0 && steps <= 64 && (steps == 0 || coef != nullptr),
              "anc_ns_batched: steps=%d out of range or null coefficients", steps);
  ANC_REQUIRE(workspace != 0 && (workspace & 255) == 0, "anc_ns_batched: workspace must be 256-byte aligned");
  const Plan pl = make_plan(workspace, E, M, N, mode, steps);
  ANC_REQUIRE(workspace_bytes >= pl.bytes, "anc_ns_batched: workspace holds %lld bytes, %lld needed",
              (long long)workspace_bytes, (long long)pl.bytes);
  hipStream_t s = anc_stream(stream);
  float *X32 = (float *)X;
  const int64_t mn = M * N;

  // ---- X /= ||X||_F + eps
  { AncProfScope prof(ANC_PROF_NS_FRO, s); hipLaunchKernelGGL(k_fro_partials, dim3((unsigned)(E * pl.nchunks)), dim3(kThreads), 0, s, X32, mn,
                     pl.nchunks, pl.partials); }
  ANC_LAUNCH_CHECK();
  { AncProfScope prof(ANC_PROF_NS_FRO, s); hipLaunchKernelGGL(k_fro_finalize, dim3((unsigned)E), dim3(kThreads), 0, s, pl.partials, pl.nchunks,
                     eps, pl.recip, (float *)nullptr); }
  ANC_LAUNCH_CHECK();
  const int64_t total8 = E * mn / 8;
  const unsigned prep_grid = (unsigned)((total8 + kThreads - 1) / kThreads);

  if (mode == ANC_NS_FP32) {
    { AncProfScope prof(ANC_PROF_NS_PREP, s); hipLaunchKernelGGL(k_ns_prep, dim3(prep_grid), dim3(kThreads), 0, s, X32, pl.recip, mn, total8,
                       (uint16_t *)nullptr, (uint16_t *)nullptr); }
    ANC_LAUNCH_CHECK();
    float *cur = X32, *nxt = pl.Yf;
    const unsigned g_mm = (unsigned)(E * (M / BM) * (M / BN)), g_mn = (unsigned)(E * (M / BM) * (N / BN));
    for (int k = 0; k < steps; ++k) {
      const float a = coef[3 * k], b = coef[3 * k + 1], c = coef[3 * k + 2];
      NsGemmF32 g{};
      g.A = cur; g.B = cur; g.K = (int)N; g.nn = 0; g.strideA = mn; g.strideB = mn;
      g.Mo = (int)M; g.No = (int)M; g.out = pl.Af; g.epi = EPI_GRAM;
      { AncProfScope prof(ANC_PROF_NS_GEMM_F32, s); hipLaunchKernelGGL(k_ns_gemm_f32, dim3(g_mm), dim3(kGemmThreads), 0, s, g); }
      ANC_LAUNCH_CHECK();
      NsGemmF32 h{};
      h.A = pl.Af; h.B = pl.Af; h.K = (int)M; h.nn = 0; h.strideA = M * M; h.strideB = M * M;
      h.Mo = (int)M; h.No = (int)M; h.cb = b; h.cc = c; h.D = pl.Af; h.out = pl.Bf; h.epi = EPI_BMAT;
      { AncProfScope prof(ANC_PROF_NS_GEMM_F32, s); hipLaunchKernelGGL(k_ns_gemm_f32, dim3(g_mm), dim3(kGemmThreads), 0, s, h); }
      ANC_LAUNCH_CHECK();
      NsGemmF32 y{};
      y.A = pl.Bf; y.B = cur; y.K = (int)M; y.nn = 1; y.strideA = M * M; y.strideB = mn;
      y.Mo = (int)M; y.No = (int)N; y.ca = a; y.D = cur; y.out = nxt; y.epi = EPI_BX;
      { AncProfScope prof(ANC_PROF_NS_GEMM_F32, s); hipLaunchKernelGGL(k_ns_gemm_f32, dim3(g_mn), dim3(kGemmThreads), 0, s, y); }
      ANC_LAUNCH_CHECK();
      float *tmp = cur; cur = nxt; nxt = tmp;
    }
    if (cur != X32)
      ANC_HIP(hipMemcpyAsync(X32, cur, (size_t)(E * mn) * sizeof(float), hipMemcpyDeviceToDevice, s));
    return ANC_OK;
  }

  // ---- bf16 matrix-core chain
  if (steps == 0) {
    { AncProfScope prof(ANC_PROF_NS_PREP, s); hipLaunchKernelGGL(k_ns_prep, dim3(prep_grid), dim3(kThreads), 0, s, X32, pl.recip, mn, total8,
                       (uint16_t *)nullptr, (uint16_t *)nullptr); }
    ANC_LAUNCH_CHECK();
    return ANC_OK;
  }
  { AncProfScope prof(ANC_PROF_NS_PREP, s); hipLaunchKernelGGL(k_ns_prep, dim3(prep_grid), dim3(kThreads), 0, s, X32, pl.recip, mn, total8,
                     pl.Xh[0], pl.Xl[0]); }
  ANC_LAUNCH_CHECK();
  ChainProb cp{pl, pl.Xh[0], pl.Xl[0], 1, nullptr, X32, E, M, N, nullptr};
  return run_bf16_chain(&cp, 1, steps, coef, force_small, s);
}

// The chain on an unnormalised bf16 pair (what anc_muon_momentum_multi_pair leaves) with the
// Frobenius partial sums already known: X0 = U / (||U|| + eps) is never materialised, the first
// step folds the scale into its epilogues.
extern "C" int anc_ns_batched_pair(uint64_t Uh, uint64_t Ul, uint64_t fro_partials, int64_t n_partials,
                                   uint64_t X32_out, int64_t E, int64_t M, int64_t N, int steps,
                                   const float *coef, float eps, int mode, uint64_t workspace,
                                   int64_t workspace_bytes, uint64_t stream) {
  const bool force_small = (mode & ANC_NS_TILE128) != 0;
  mode &= ~ANC_NS_TILE128;
  if (int rc = check_shape(E, M, N, mode, "anc_ns_batched_pair")) return rc;
  ANC_REQUIRE(mode != ANC_NS_FP32, "anc_ns_batched_pair: the fp32 chain takes fp32 input (anc_ns_batched)");
  ANC_REQUIRE(Uh != 0 && Ul != 0 && ((Uh | Ul) & 15) == 0 && X32_out != 0 && (X32_out & 15) == 0,
              "anc_ns_batched_pair: pointers must be 16-byte aligned and non-null");
  ANC_REQUIRE(fro_partials != 0 && n_partials > 0 && n_partials < (1 << 30),
              "anc_ns_batched_pair: need the Frobenius partial sums (n_partials per matrix)");
  ANC_REQUIRE(steps >= 2 && steps <= 64 && coef != nullptr,
              "anc_ns_batched_pair: steps=%d: needs at least 2 steps (the fp32 result may overlay the input pair)", steps);
  ANC_REQUIRE(workspace != 0 && (workspace & 255) == 0, "anc_ns_batched_pair: workspace must be 256-byte aligned");
  const Plan pl = make_plan(workspace, E, M, N, mode, steps);
  ANC_REQUIRE(workspace_bytes >= pl.bytes, "anc_ns_batched_pair: workspace holds %lld bytes, %lld needed",
              (long long)workspace_bytes, (long long)pl.bytes);
  hipStream_t s = anc_stream(stream);
  { AncProfScope prof(ANC_PROF_NS_FRO, s); hipLaunchKernelGGL(k_fro_finalize, dim3((unsigned)E), dim3(kThreads), 0, s,
                     (const double *)fro_partials, (int)n_partials, eps, pl.recip, pl.pow2); }
  ANC_LAUNCH_CHECK();
  { AncProfScope prof(ANC_PROF_NS_FRO, s); hipLaunchKernelGGL(k_pair_rescale, dim3((unsigned)E), dim3(kThreads), 0, s,
                     (uint16_t *)Uh, (uint16_t *)Ul, pl.pow2, M * N); }
  ANC_LAUNCH_CHECK();
  ChainProb cp{pl, (const uint16_t *)Uh, (const uint16_t *)Ul, 0, pl.recip, (float *)X32_out, E, M, N, nullptr};
  return run_bf16_chain(&cp, 1, steps, coef, force_small, s);
}

// n_probs <= 8 independent batches (the shape groups of one optimizer step) through the chain
// side by side: each product of each step is one launch over all of them, which keeps the
// CUs busy where per-batch launches would each end in a partly filled last wave. Same
// results, bit for bit, as anc_ns_batched_pair on each batch. All dims multiples of 256.
static int pair_multi_impl(const char *who, const anc_ns_problem_t *probs, int32_t n_probs,
                           const uint64_t *desc_tables, const NsUpdate *upd, int steps, const float *coef,
                           float eps, int mode, uint64_t stream) {
  ANC_REQUIRE(probs != nullptr && n_probs >= 1 && n_probs <= kMaxGroups, "%s: 1..%d problems", who, kMaxGroups);
  ANC_REQUIRE(mode == ANC_NS_BF16 || mode == ANC_NS_BF16_FAST || mode == ANC_NS_BF16_X3 || mode == ANC_NS_BF16_LATE3,
              "%s: bf16 modes only", who);
  ANC_REQUIRE(steps >= 2 && steps <= 64 && coef != nullptr, "%s: steps=%d: 2..64", who, steps);
  hipStream_t s = anc_stream(stream);
  ChainProb cp[kMaxGroups];
  int order[kMaxGroups];
  for (int q = 0; q < n_probs; ++q) {
    const anc_ns_problem_t &b = probs[q];
    if (int rc = check_shape(b.E, b.M, b.N, mode, who)) return rc;
    ANC_REQUIRE(b.M % 256 == 0 && b.N % 256 == 0, "%s: dims must be multiples of 256", who);
    ANC_REQUIRE(b.Uh != 0 && b.Ul != 0 && ((b.Uh | b.Ul | b.X32_out) & 15) == 0,
                "%s: pointers must be 16-byte aligned and non-null", who);
    if (desc_tables == nullptr) ANC_REQUIRE(b.X32_out != 0, "%s: null X32_out", who);
    else ANC_REQUIRE(desc_tables[q] != 0 && (desc_tables[q] & 7) == 0, "%s: null or misaligned descriptor table", who);
    ANC_REQUIRE(b.fro_partials != 0 && b.n_partials > 0 && b.n_partials < (1 << 30),
                "%s: need the Frobenius partial sums", who);
    ANC_REQUIRE(b.workspace != 0 && (b.workspace & 255) == 0, "%s: workspace must be 256-byte aligned", who);
    order[q] = q;
  }
  // longest tiles first: by N (the Gram product's K), then by M
  for (int a = 0; a < n_probs; ++a)
    for (int c = a + 1; c < n_probs; ++c) {
      const anc_ns_problem_t &x = probs[order[a]], &y = probs[order[c]];
      if (y.N > x.N || (y.N == x.N && y.M > x.M)) { const int t = order[a]; order[a] = order[c]; order[c] = t; }
    }
  for (int q = 0; q < n_probs; ++q) {
    const anc_ns_problem_t &b = probs[order[q]];
    const Plan pl = make_plan(b.workspace, b.E, b.M, b.N, mode, steps);
    ANC_REQUIRE(b.workspace_bytes >= pl.bytes, "%s: workspace holds %lld bytes, %lld needed", who,
                (long long)b.workspace_bytes, (long long)pl.bytes);
    { AncProfScope prof(ANC_PROF_NS_FRO, s); hipLaunchKernelGGL(k_fro_finalize, dim3((unsigned)b.E), dim3(kThreads), 0, s,
                       (const double *)b.fro_partials, (int)b.n_partials, eps, pl.recip, pl.pow2); }
    ANC_LAUNCH_CHECK();
    { AncProfScope prof(ANC_PROF_NS_FRO, s); hipLaunchKernelGGL(k_pair_rescale, dim3((unsigned)b.E), dim3(kThreads), 0, s,
                       (uint16_t *)b.Uh, (uint16_t *)b.Ul, pl.pow2, b.M * b.N); }
    ANC_LAUNCH_CHECK();
    cp[q] = ChainProb{pl, (const uint16_t *)b.Uh, (const uint16_t *)b.Ul, 0, pl.recip, (float *)b.X32_out, b.E, b.M, b.N,
                      desc_tables ? (const anc_muon_desc_t *)desc_tables[order[q]] : nullptr};
  }
  return run_bf16_chain(cp, n_probs, steps, coef, false, s, upd);
}

extern "C" int anc_ns_batched_pair_multi(const anc_ns_problem_t *probs, int32_t n_probs, int steps,
                                         const float *coef, float eps, int mode, uint64_t stream) {
  return pair_multi_impl("anc_ns_batched_pair_multi", probs, n_probs, nullptr, nullptr, steps, coef, eps, mode, stream);
}

// The same chain with the Muon weight update applied by the last step's epilogue: problem q's
// matrix e is the orthogonalised update of the weight desc_tables[q][e] (p32, p16, K, N,
// transpose, scale_idx and seed are read; p16t must be 0). Same bits in p32 and p16 as the chain
// followed by anc_muon_update_multi, without the fp32 hand-off in between.
extern "C" int anc_muon_ns_update_multi(const anc_ns_problem_t *probs, int32_t n_probs,
                                        const uint64_t *desc_tables, int steps, const float *coef, float eps,
                                        int mode, const float *lr_scales, int sr, uint32_t seed_base,
                                        uint64_t ctl, uint64_t stream) {
  ANC_REQUIRE(desc_tables != nullptr && lr_scales != nullptr, "anc_muon_ns_update_multi: null descriptor tables or lr_scales");
  NsUpdate u{};
  for (int k = 0; k < ANC_MUON_MAX_SCALES; ++k) u.lr[k] = lr_scales[k];
  ANC_REQUIRE(sr == 0 || sr == ANC_SR_ON || sr == (ANC_SR_ON | ANC_SR_STEP_SEED),
              "anc_muon_ns_update_multi: sr must be 0, ANC_SR_ON or ANC_SR_ON | ANC_SR_STEP_SEED");
  ANC_REQUIRE(!(sr & ANC_SR_STEP_SEED) || ctl != 0, "anc_muon_ns_update_multi: ANC_SR_STEP_SEED needs the control block");
  u.sr = sr;
  u.seed_base = seed_base;
  u.ctl = (const anc_step_ctl_t *)ctl;
  return pair_multi_impl("anc_muon_ns_update_multi", probs, n_probs, desc_tables, &u, steps, coef, eps, mode, stream);
}
