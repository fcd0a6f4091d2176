// MXFP8 re-quantisation of the bf16 weights the optimizer step has just refreshed.
//
// Replaces `_quant_mxfp8_w` and `_quant_mxfp8_w_cm` (ancora/kernels/quant.py:60-100), which the
// reference launches from the next forward once the step has set its dirty flags
// (ancora/model/resident_train.py:190-199, 354-357). Per block of 32 consecutive K and per
// column: amax of |w|, E8M0 scale byte = (biased fp32 exponent of amax) - 7 (0 below 7), element
// = E4M3FN(w / 2^(byte-127)), round to nearest even. All of it is integer arithmetic on the bf16
// bit patterns: an element with biased exponent eb and 7-bit mantissa m becomes the E4M3 number
// with biased exponent e = eb - byte + 7 and mantissa m rounded to 3 bits (carry into e),
// or, for e <= 0, the multiple of 2^-9 nearest to 1.m * 2^(e-7).
//
// HBM-bound byte work: 2 B read, 1 + 1/32 B written per element. A lane loads 16 rows x 8 columns
// with 16-byte loads; the stores of either output layout fill whole 128-byte lines: row-major
// (K,N) rows of 8 bytes per lane over 16 lanes, or column-major (N,K) 16 bytes per lane and
// column, the 8 lanes that hold the 128 rows of the tile completing the line.
#include "common.h"

namespace {

constexpr int kThreads = 256;
constexpr int kRows = 32;          // scale block along K
constexpr int kHalf = 16;          // rows of it held by one lane

// E4M3FN byte (without sign) of the bf16 magnitude `a` (15 bits) scaled by 2^(127-byte);
// adj = (7 - byte) << 7.
__device__ __forceinline__ uint32_t e4m3_general(uint32_t a, int adj) {
  if (a >= 0x7F80u) return 0x7Fu;                  // Inf / NaN
  if (a < 0x80u) return 0u;                        // zero and bf16 subnormals
  const int t = (int)a + adj;                      // (e << 7) | m
  if (t >= 128) return (uint32_t)(t + 7 + ((t >> 4) & 1)) >> 4;
  const int sh = 5 - (t >> 7);                     // bits of the 8-bit significand to drop (>= 5)
  if (sh >= 10) return 0u;
  const uint32_t sig = 0x80u | (a & 0x7Fu);
  return (sig + (1u << (sh - 1)) - 1u + ((sig >> sh) & 1u)) >> sh;
}

// Wavefront tile: 64 rows x 128 columns (row-major output) or 128 rows x 64 columns (column-major
// output). A lane holds 16 rows x 8 columns, i.e. half a scale block; the two halves sit in lanes
// `lane` and `lane ^ kPartner` and exchange their column maxima.
template <bool CM>
__global__ void __launch_bounds__(kThreads, 4)
k_quant_mxfp8_w(const uint16_t *__restrict__ w, uint8_t *__restrict__ fp8, uint8_t *__restrict__ sc,
                int K, int N, int64_t tiles) {
  constexpr int kColGroups = CM ? 8 : 16;          // lanes across the columns (8 columns each)
  constexpr int kTileCols = kColGroups * 8, kTileRows = (64 / kColGroups) * kHalf;
  const int lane = threadIdx.x & 63;
  const int64_t tile = (int64_t)blockIdx.x * (kThreads / 64) + (threadIdx.x >> 6);
  if (tile >= tiles) return;                                      // whole wavefront
  const int tn = N / kTileCols, tk = K / kTileRows;
  const int cb = (int)(tile % tn);
  const int rb = (int)((tile / tn) % tk);
  const int64_t e = tile / ((int64_t)tn * tk);
  const int hb = lane / kColGroups, half = hb & 1;                // half-block of this lane
  const int kb = rb * (kTileRows / kRows) + (hb >> 1);            // scale block along K
  const int col0 = cb * kTileCols + (lane % kColGroups) * 8;
  const int row0 = kb * kRows + half * kHalf;
  const uint16_t *src = w + (e * K + row0) * N + col0;

  anc_u32x4 v[kHalf];
#pragma unroll
  for (int r = 0; r < kHalf; ++r) v[r] = anc_ld_stream((const anc_u32x4 *)(src + (int64_t)r * N));

  // amax per column as the maximum of the 15-bit magnitudes (same order as the values), two
  // columns per packed 16-bit max
  typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));
  u16x2 am2[4] = {{0, 0}, {0, 0}, {0, 0}, {0, 0}};
#pragma unroll
  for (int r = 0; r < kHalf; ++r) {
    const uint32_t q[4] = {v[r].x, v[r].y, v[r].z, v[r].w};
#pragma unroll
    for (int h = 0; h < 4; ++h) {
      const uint32_t m = q[h] & 0x7FFF7FFFu;
      am2[h] = __builtin_elementwise_max(am2[h], __builtin_bit_cast(u16x2, m));
    }
  }
  uint32_t amax[8];
#pragma unroll
  for (int h = 0; h < 4; ++h) {
    uint32_t m = __builtin_bit_cast(uint32_t, am2[h]);
    const uint32_t o = (uint32_t)__shfl_xor((int)m, kColGroups, 64);
    m = __builtin_bit_cast(uint32_t, __builtin_elementwise_max(am2[h], __builtin_bit_cast(u16x2, o)));
    amax[2 * h] = m & 0xFFFFu;
    amax[2 * h + 1] = m >> 16;
  }
  uint32_t byte[8];
  int adj[8];
  bool plain = true;      // every column: finite, and a scale byte high enough that an element
                          // with a zero exponent field cannot reach the normal range
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const uint32_t ea = amax[j] >> 7;
    byte[j] = ea >= 7u ? ea - 7u : 0u;
    adj[j] = (7 - (int)byte[j]) * 128;
    plain = plain && ea != 255u && byte[j] >= 8u;
  }

  // scale bytes, from the lane that holds the first half of the block
  if (half == 0) {
    if constexpr (!CM) {
      const anc_u32x2 s2 = {byte[0] | (byte[1] << 8) | (byte[2] << 16) | (byte[3] << 24),
                            byte[4] | (byte[5] << 8) | (byte[6] << 16) | (byte[7] << 24)};
      anc_st_stream((anc_u32x2 *)(sc + (e * (K / kRows) + kb) * N + col0), s2);
    } else {
#pragma unroll
      for (int j = 0; j < 8; ++j) sc[(e * N + col0 + j) * (int64_t)(K / kRows) + kb] = (uint8_t)byte[j];
    }
  }

  if constexpr (!CM) {
    // row-major: 8 bytes per row
#pragma unroll
    for (int r = 0; r < kHalf; ++r) {
      const uint32_t q[4] = {v[r].x, v[r].y, v[r].z, v[r].w};
      uint32_t b[8];
      bool fast = plain;
      int t[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const uint32_t a = ((j & 1) ? (q[j >> 1] >> 16) : q[j >> 1]) & 0x7FFFu;
        t[j] = (int)a + adj[j];
        fast = fast && t[j] >= 128;
      }
      if (fast) {                                 // normal E4M3 range: round the mantissa to 3 bits
#pragma unroll
        for (int j = 0; j < 8; ++j) b[j] = (uint32_t)(t[j] + 7 + ((t[j] >> 4) & 1)) >> 4;
      } else {
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const uint32_t a = ((j & 1) ? (q[j >> 1] >> 16) : q[j >> 1]) & 0x7FFFu;
          b[j] = e4m3_general(a, adj[j]);
        }
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) b[j] |= ((j & 1) ? (q[j >> 1] >> 24) : (q[j >> 1] >> 8)) & 0x80u;
      const anc_u32x2 o = {b[0] | (b[1] << 8) | (b[2] << 16) | (b[3] << 24),
                           b[4] | (b[5] << 8) | (b[6] << 16) | (b[7] << 24)};
      anc_st_stream((anc_u32x2 *)(fp8 + (e * K + row0 + r) * N + col0), o);
      __builtin_amdgcn_sched_barrier(0);          // one row at a time: keeps the live set small
    }
  } else {
    // column-major: 16 bytes (the lane's 16 rows) per column
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      uint32_t word[kHalf];
      int t[kHalf];
      bool fast = plain;
#pragma unroll
      for (int r = 0; r < kHalf; ++r) {
        const uint32_t q[4] = {v[r].x, v[r].y, v[r].z, v[r].w};
        word[r] = (j & 1) ? (q[j >> 1] >> 16) : (q[j >> 1] & 0xFFFFu);
        t[r] = (int)(word[r] & 0x7FFFu) + adj[j];
        fast = fast && t[r] >= 128;
      }
      uint32_t o[4] = {0, 0, 0, 0};
#pragma unroll
      for (int r = 0; r < kHalf; ++r) {
        uint32_t b;
        if (fast) b = (uint32_t)(t[r] + 7 + ((t[r] >> 4) & 1)) >> 4;
        else      b = e4m3_general(word[r] & 0x7FFFu, adj[j]);
        b |= (word[r] >> 8) & 0x80u;
        o[r >> 2] |= b << (8 * (r & 3));
      }
      const anc_u32x4 o4 = {o[0], o[1], o[2], o[3]};
      anc_st_stream((anc_u32x4 *)(fp8 + (e * N + col0 + j) * (int64_t)K + row0), o4);
      __builtin_amdgcn_sched_barrier(0);          // one column at a time
    }
  }
}

}  // namespace

extern "C" int anc_quant_mxfp8_w(uint64_t w_bf16, uint64_t fp8_out, uint64_t scale_out, int64_t E,
                                 int64_t K, int64_t N, int col_major, uint64_t stream) {
  ANC_REQUIRE(w_bf16 && fp8_out && scale_out && E > 0, "anc_quant_mxfp8_w: bad arguments");
  ANC_REQUIRE(K > 0 && N > 0 && K % 128 == 0 && N % 128 == 0,
              "anc_quant_mxfp8_w: K=%lld and N=%lld must be positive multiples of 128", (long long)K,
              (long long)N);
  ANC_REQUIRE(K < (1ll << 31) && N < (1ll << 31), "anc_quant_mxfp8_w: dimension too large");
  ANC_REQUIRE(((w_bf16 | fp8_out) & 15) == 0 && (scale_out & 7) == 0,
              "anc_quant_mxfp8_w: w and fp8_out must be 16-byte, scale_out 8-byte aligned");
  const int64_t tiles = E * (K * N / 8192);                       // 64x128 or 128x64 per wavefront
  const int64_t blocks = (tiles + kThreads / 64 - 1) / (kThreads / 64);
  ANC_REQUIRE(blocks < (1ll << 31), "anc_quant_mxfp8_w: too large");
  hipStream_t s = anc_stream(stream);
  AncProfScope prof(ANC_PROF_MISC, s);
  if (col_major)
    hipLaunchKernelGGL((k_quant_mxfp8_w<true>), dim3((unsigned)blocks), dim3(kThreads), 0, s,
                       (const uint16_t *)w_bf16, (uint8_t *)fp8_out, (uint8_t *)scale_out, (int)K, (int)N, tiles);
  else
    hipLaunchKernelGGL((k_quant_mxfp8_w<false>), dim3((unsigned)blocks), dim3(kThreads), 0, s,
                       (const uint16_t *)w_bf16, (uint8_t *)fp8_out, (uint8_t *)scale_out, (int)K, (int)N, tiles);
  ANC_LAUNCH_CHECK();
  return ANC_OK;
}
