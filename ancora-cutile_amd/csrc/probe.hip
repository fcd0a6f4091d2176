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

}  // namespace

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
