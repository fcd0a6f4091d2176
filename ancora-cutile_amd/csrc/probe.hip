// Hardware probe behind the roofline discussion of the Newton-Schulz GEMM: the rate of
// v_mfma_f32_32x32x16_bf16 on register operands while the same wavefronts also issue LDS
// fragment reads (ds_read_b128) and LDS-DMA loads (global_load_lds_dwordx4) that nothing
// depends on, in the proportions of the GEMM's K loop (8 wavefronts per CU, per wavefront and
// iteration 16 matrix instructions, `nread` LDS reads, `ndma` DMA instructions of 1 KiB). It
// answers what the matrix pipe sustains next to that much unrelated traffic, i.e. the ceiling
// of any kernel with this data flow, whatever its schedule. No reference counterpart.
#include "ns_common.h"

namespace {

__device__ __forceinline__ void probe_dma16(const void *g, uint32_t lds_base) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(lds_base), "v"(g)
               : "memory", "m0");
}

template <int NREAD, int NDMA>
__global__ void __launch_bounds__(512) k_probe_mfma_mix(int iters, const char *src, size_t span, int hbm,
                                                        float *sink) {
  __shared__ __attribute__((aligned(1024))) unsigned char lds[131072];
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  for (int i = threadIdx.x; i < 131072 / 4; i += 512) ((uint32_t *)lds)[i] = i;
  __syncthreads();
  f32x16 acc[8];
  for (int i = 0; i < 8; ++i)
    for (int r = 0; r < 16; ++r) acc[i][r] = 0.f;
  bf16x8 a, b;
  for (int i = 0; i < 8; ++i) {
    a[i] = (__bf16)(float)(lane + i);
    b[i] = (__bf16)(float)(lane * 3 + i);
  }
  anc_u32x4 x = {0, 0, 0, 0};
  const unsigned char *rbase = lds + lane * 16;          // conflict-free reads in the first 64 KiB
  const uint32_t dbase =
      (uint32_t)(uintptr_t)((__attribute__((address_space(3))) void *)(lds + 65536 + wave * 8192));
  // 64 KiB per workgroup: stays in L2 unless `hbm` makes every iteration move on by 16 MiB
  size_t goff = ((size_t)blockIdx.x * 65536 + wave * 8192 + lane * 16) % span;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int d = 0; d < NDMA; ++d) probe_dma16(src + goff + d * 1024, dbase + d * 1024);
    if (hbm) {
      goff += (size_t)256 * 65536;
      if (goff >= span) goff -= span;
    }
#pragma unroll
    for (int f = 0; f < NREAD; ++f) x ^= *(const anc_u32x4 *)(rbase + ((f * 1024 + wave * 2048) & 65535));
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int i = 0; i < 8; ++i) acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc[i], 0, 0, 0);
    if (NDMA) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
  }
  float s = 0;
  for (int i = 0; i < 8; ++i) s += acc[i][0];
  if (s == 12345.f || x[0] == 0x1234567u) sink[threadIdx.x] = s;
}

template <int NREAD, int NDMA>
void launch(int iters, const char *src, size_t span, int hbm, float *sink, hipStream_t s) {
  hipLaunchKernelGGL((k_probe_mfma_mix<NREAD, NDMA>), dim3(256), dim3(512), 0, s, iters, src, span, hbm, sink);
}

// ---- K-loop probe ------------------------------------------------------------------------
// The GEMM's K loop by itself: 256x256x32 tiles, 8 wavefronts x (128x64) or 4 x (128x128), the
// 4-stage LDS-DMA ring with the DMA instructions interleaved between the matrix instructions, real
// fragment reads feeding the MFMAs, one barrier per K tile -- and nothing else: no epilogue, and
// every workgroup multiplies the same two 256-row operands, so that every operand load hits in
// cache. What this reaches is what the loop structure can do when memory is out of the way.
template <int N> __device__ __forceinline__ void probe_wait_vm() {
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}
__device__ __forceinline__ void probe_lds_barrier() {
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_waitcnt(0xC07F);
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}

template <int NWM, int NWN, int WM, int WN>
__global__ void __launch_bounds__(NWM * NWN * 64, 1)
k_probe_kloop(const uint16_t *A0, int64_t group_stride, int share, int ldk, int nk, int reps, float *sink) {
  constexpr int TM = 256, TN = 256, ROWB = 64, NS = 4, kStage = (TM + TN) * ROWB;
  constexpr int NW = NWM * NWN;
  constexpr int IPS = (TM + TN) / 16 / NW, IA = TM / 16 / NW, NM = WM * WN;
  static_assert(NWM * WM * 32 == TM && NWN * WN * 32 == TN, "tile");
  __shared__ __attribute__((aligned(1024))) unsigned char lds[NS * kStage];
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wm = wave / NWN, wn = wave % NWN;
  // `share` workgroups of one XCD (workgroup b runs on XCD b % 8) multiply the same operands
  const int group = ((int)blockIdx.x % 8) * (32 / share) + ((int)blockIdx.x / 8) / share;
  const uint16_t *A = A0 + (int64_t)group * group_stride, *B = A + (int64_t)256 * ldk;
  const int lrow = lane >> 2, pch = lane & 3;
  const uint32_t voff = (uint32_t)(lrow * ldk * 2 + ((pch ^ ((lrow >> 2) & 3)) * 16));
  const char *gA = (const char *)A + (int64_t)(wave * IA * 16) * ldk * 2;
  const char *gB = (const char *)B + (int64_t)(wave * (IPS - IA) * 16) * ldk * 2;
  int kt_issue = 0;
  auto lds_of = [&](const void *q) { return (uint32_t)(uintptr_t)((__attribute__((address_space(3))) const void *)q); };
  auto issue_piece = [&](int i, int stage) {
    unsigned char *st = lds + stage * kStage;
    if (i < IA)
      probe_dma16(gA + (int64_t)(i * 16) * ldk * 2 + kt_issue * ROWB + voff, lds_of(st + (wave * IA + i) * 1024));
    else
      probe_dma16(gB + (int64_t)((i - IA) * 16) * ldk * 2 + kt_issue * ROWB + voff,
                  lds_of(st + TM * ROWB + (wave * (IPS - IA) + (i - IA)) * 1024));
  };
  auto advance = [&]() { if (++kt_issue == nk) kt_issue = 0; };
  const int a_base = (wm * WM * 32 + (lane & 31)) * ROWB, b_base = TM * ROWB + (wn * WN * 32 + (lane & 31)) * ROWB;
  int swz[2];
  for (int kk = 0; kk < 2; ++kk) swz[kk] = ((kk * 2 + (lane >> 5)) ^ ((lane >> 2) & 3)) * 16;
  struct Fr { bf16x8 a[WM], b[WN]; };
  auto frags = [&](int stage, int kk, Fr &f) {
    const unsigned char *st = lds + stage * kStage;
#pragma unroll
    for (int i = 0; i < WM; ++i) f.a[i] = *(const bf16x8 *)(st + a_base + i * 32 * ROWB + swz[kk]);
#pragma unroll
    for (int j = 0; j < WN; ++j) f.b[j] = *(const bf16x8 *)(st + b_base + j * 32 * ROWB + swz[kk]);
  };
  f32x16 acc[WM][WN];
#pragma unroll
  for (int i = 0; i < WM; ++i)
#pragma unroll
    for (int j = 0; j < WN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
  const int total = nk * reps;                       // a multiple of NS
  Fr f[2];
#pragma unroll
  for (int s = 0; s < NS - 1; ++s) {
    for (int i = 0; i < IPS; ++i) issue_piece(i, s);
    advance();
  }
  probe_wait_vm<(NS - 2) * IPS>();
  probe_lds_barrier();
  frags(0, 0, f[0]);
  for (int step = 0; step < total; step += NS) {
#pragma unroll
    for (int s0 = 0; s0 < NS; ++s0) {
      const int cur = s0, nxt = (s0 + 1) % NS, fill = (s0 + NS - 1) % NS;
      frags(cur, 1, f[1]);
#pragma unroll
      for (int idx = 0; idx < NM; ++idx) {
        acc[idx / WN][idx % WN] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(f[0].a[idx / WN], f[0].b[idx % WN],
                                                                          acc[idx / WN][idx % WN], 0, 0, 0);
#pragma unroll
        for (int i = 0; i < IPS; ++i)
          if (((i + 1) * NM + IPS - 1) / IPS - 1 == idx) {
            __builtin_amdgcn_sched_barrier(0);
            issue_piece(i, fill);
            __builtin_amdgcn_sched_barrier(0);
          }
      }
      advance();
      probe_wait_vm<(NS - 2) * IPS>();
      probe_lds_barrier();
      frags(nxt, 0, f[0]);
#pragma unroll
      for (int idx = 0; idx < NM; ++idx)
        acc[idx / WN][idx % WN] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(f[1].a[idx / WN], f[1].b[idx % WN],
                                                                          acc[idx / WN][idx % WN], 0, 0, 0);
    }
  }
  probe_wait_vm<0>();
  float s = 0;
#pragma unroll
  for (int i = 0; i < WM; ++i)
#pragma unroll
    for (int j = 0; j < WN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) s += acc[i][j][r];
  if (s == 12345.678f) sink[threadIdx.x] = s;
}

}  // namespace

extern "C" int anc_probe_kloop(int waves, int share, int k_tiles, int reps, uint64_t src, int64_t span_bytes,
                               uint64_t sink, double *tflops) {
  ANC_REQUIRE(waves == 8 || waves == 4, "anc_probe_kloop: 8 or 4 wavefronts per workgroup");
  ANC_REQUIRE(share == 1 || share == 2 || share == 4 || share == 8 || share == 16 || share == 32,
              "anc_probe_kloop: share must be a power of two in 1..32");
  ANC_REQUIRE(k_tiles >= 4 && k_tiles % 4 == 0 && k_tiles <= 4096 && reps >= 1 && reps <= 4096,
              "anc_probe_kloop: k_tiles must be a multiple of 4 in 4..4096, reps in 1..4096");
  const int ldk = k_tiles * 32;
  const int64_t group_stride = 2ll * 256 * ldk;                       // elements: A then B
  const int groups = 256 / share;
  ANC_REQUIRE(src != 0 && (src & 15) == 0 && span_bytes >= groups * group_stride * 2 && sink != 0 && tflops != nullptr,
              "anc_probe_kloop: need a source buffer of (256 / share) x 2 x 256 x 32*k_tiles bf16 and a 2 KiB sink");
  const uint16_t *A = (const uint16_t *)src;
  hipEvent_t e0, e1;
  ANC_HIP(hipEventCreate(&e0));
  ANC_HIP(hipEventCreate(&e1));
  for (int pass = 0; pass < 2; ++pass) {           // pass 0 warms the clocks and the caches
    const int r = pass ? reps : 1;
    ANC_HIP(hipEventRecord(e0, 0));
    if (waves == 8)
      hipLaunchKernelGGL((k_probe_kloop<2, 4, 4, 2>), dim3(256), dim3(512), 0, 0, A, group_stride, share, ldk, k_tiles, r, (float *)sink);
    else
      hipLaunchKernelGGL((k_probe_kloop<2, 2, 4, 4>), dim3(256), dim3(256), 0, 0, A, group_stride, share, ldk, k_tiles, r, (float *)sink);
    ANC_LAUNCH_CHECK();
    ANC_HIP(hipEventRecord(e1, 0));
    ANC_HIP(hipEventSynchronize(e1));
  }
  float ms = 0.f;
  ANC_HIP(hipEventElapsedTime(&ms, e0, e1));
  ANC_HIP(hipEventDestroy(e0));
  ANC_HIP(hipEventDestroy(e1));
  *tflops = 256.0 * 2.0 * 256 * 256 * 32 * (double)k_tiles * reps / (ms * 1e-3) / 1e12;
  return ANC_OK;
}

extern "C" int anc_probe_mfma_mix(int nread, int ndma, int hbm, int iters, uint64_t src, int64_t span_bytes,
                                  uint64_t sink, double *tflops, double *cycles_per_iter) {
  ANC_REQUIRE(src != 0 && (src & 15) == 0 && span_bytes >= (64ll << 20) && sink != 0 && iters > 0,
              "anc_probe_mfma_mix: need a source buffer of at least 64 MiB and a 2 KiB sink");
  ANC_REQUIRE(tflops != nullptr && cycles_per_iter != nullptr, "anc_probe_mfma_mix: null outputs");
  const int sel = nread * 100 + ndma;
  ANC_REQUIRE(sel == 0 || sel == 1200 || sel == 4 || sel == 1204 || sel == 2408,
              "anc_probe_mfma_mix: (nread, ndma) must be one of (0,0) (12,0) (0,4) (12,4) (24,8)");
  hipEvent_t e0, e1;
  ANC_HIP(hipEventCreate(&e0));
  ANC_HIP(hipEventCreate(&e1));
  for (int pass = 0; pass < 2; ++pass) {           // pass 0 warms the clocks and the L2
    const int n = pass ? iters : (iters < 2000 ? iters : 2000);
    ANC_HIP(hipEventRecord(e0, 0));
    switch (sel) {
      case 0: launch<0, 0>(n, (const char *)src, (size_t)span_bytes, hbm, (float *)sink, 0); break;
      case 1200: launch<12, 0>(n, (const char *)src, (size_t)span_bytes, hbm, (float *)sink, 0); break;
      case 4: launch<0, 4>(n, (const char *)src, (size_t)span_bytes, hbm, (float *)sink, 0); break;
      case 1204: launch<12, 4>(n, (const char *)src, (size_t)span_bytes, hbm, (float *)sink, 0); break;
      default: launch<24, 8>(n, (const char *)src, (size_t)span_bytes, hbm, (float *)sink, 0); break;
    }
    ANC_LAUNCH_CHECK();
    ANC_HIP(hipEventRecord(e1, 0));
    ANC_HIP(hipEventSynchronize(e1));
  }
  float ms = 0.f;
  ANC_HIP(hipEventElapsedTime(&ms, e0, e1));
  ANC_HIP(hipEventDestroy(e0));
  ANC_HIP(hipEventDestroy(e1));
  const double flops = 256.0 * 8 * (double)iters * 16 * 2.0 * 32 * 32 * 16;
  *tflops = flops / (ms * 1e-3) / 1e12;
  *cycles_per_iter = 1024.0 * 2500.0 / *tflops;   // 16 MFMAs x 2 wavefronts per SIMD take 1024 cycles at the 2.5 PFLOP/s rate
  return ANC_OK;
}
