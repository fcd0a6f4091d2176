// Fixed-order sum of squares over one 8192-element chunk: the building block of the
// global gradient norm and of the per-matrix Frobenius norm.
//   for j in 0..3: lane t takes the 8 consecutive elements of vector j*256 + t, adds
//     their squares left to right in fp32 (a bf16 square is exact in fp32), widens the
//     8-sum to fp64 and adds it to its fp64 accumulator;
//   the 64 lanes of a wavefront are combined by an xor butterfly (32,16,...,1);
//   the 4 wavefront sums are added in wavefront order.
// Elements at or past n count as zero.
#pragma once
#include "common.h"

namespace anc_reduce {

constexpr int kThreads = 256;
constexpr int kRun = 8;                                   // elements per lane per access
constexpr int kIters = ANC_GN_CHUNK / (kThreads * kRun);  // 4
static_assert(kIters * kThreads * kRun == ANC_GN_CHUNK, "chunk must split evenly");

template <int GD>
__device__ __forceinline__ float run_sumsq(const void *g, int64_t e, int64_t n) {
  float x[kRun];
  if (e + kRun <= n) {
    if (GD == ANC_BF16) {
      const anc_u32x4 r = anc_ld_stream((const anc_u32x4 *)((const uint16_t *)g + e));
      const uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        x[2 * k] = __uint_as_float(w[k] << 16);
        x[2 * k + 1] = __uint_as_float(w[k] & 0xFFFF0000u);
      }
    } else {
      const anc_f32x4 a = anc_ld_stream((const anc_f32x4 *)((const float *)g + e));
      const anc_f32x4 b = anc_ld_stream((const anc_f32x4 *)((const float *)g + e + 4));
      x[0] = a.x; x[1] = a.y; x[2] = a.z; x[3] = a.w;
      x[4] = b.x; x[5] = b.y; x[6] = b.z; x[7] = b.w;
    }
  } else {
#pragma unroll
    for (int k = 0; k < kRun; ++k) {
      float val = 0.0f;
      if (e + k < n) {
        if (GD == ANC_BF16) val = anc_bf16_bits_to_f32(((const uint16_t *)g)[e + k]);
        else                val = ((const float *)g)[e + k];
      }
      x[k] = val;
    }
  }
  float s = x[0] * x[0];
#pragma unroll
  for (int k = 1; k < kRun; ++k) s = s + x[k] * x[k];
  return s;
}

// The chunk's partial from the kIters run sums of every lane (s[j]: run j*kThreads + lane).
__device__ __forceinline__ void chunk_finish(const float (&s)[kIters], double *__restrict__ out) {
  __shared__ double wave_sum[kThreads / 64];
  double acc = 0.0;
#pragma unroll
  for (int j = 0; j < kIters; ++j) acc = acc + (double)s[j];
  acc = anc_wave_sum_f64(acc);
  if ((threadIdx.x & 63) == 0) wave_sum[threadIdx.x >> 6] = acc;
  __syncthreads();
  if (threadIdx.x == 0) {
    double t = wave_sum[0];
#pragma unroll
    for (int w = 1; w < kThreads / 64; ++w) t = t + wave_sum[w];
    *out = t;
  }
}

template <int GD>
__device__ __forceinline__ void chunk_partial(const void *g, int64_t n, int64_t chunk,
                                              double *__restrict__ out) {
  const int64_t base = chunk * (int64_t)ANC_GN_CHUNK;
  float s[kIters];
#pragma unroll
  for (int j = 0; j < kIters; ++j) {
    const int64_t e = base + ((int64_t)j * kThreads + threadIdx.x) * kRun;
    s[j] = (e < n) ? run_sumsq<GD>(g, e, n) : 0.0f;
  }
  chunk_finish(s, out);
}

}  // namespace anc_reduce
